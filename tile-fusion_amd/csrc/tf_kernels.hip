// HIP kernels of libtilefusion_hip, written for gfx950 (CDNA4): 64-wide wavefronts,
// LDS slabs of the intermediate, fp32 MFMA for the tile GEMM.
//
// Work decomposition used by every sparse kernel here: a wavefront is cut into lane
// groups of LPR lanes; one group owns one output row at a time and each lane owns VEC
// adjacent columns of it (LPR*VEC columns per pass, a 16-byte load per lane when
// VEC = 4).  A group first loads up to LPR (column, value) pairs of its CSR row with
// one coalesced load, then walks them in CSR order, broadcasting each pair inside the
// group, so the per-element sequence is acc = fma(value, x[column], acc) exactly as in
// the reference's AVX2 kernels (fusion/src/SpMM_SpMM_vectorized.cpp:892-936).
#include <hip/hip_runtime.h>
#include <climits>
#include <type_traits>

#include "tf_internal.h"
#include "tf_device.h"

namespace tf {


// ---------------------------------------------------------------------------------
// Fused SpMM-SpMM tile kernel: one workgroup per tile.
//   phase 1  T[r,:] = sum_j Bx[j] * C[Bi[j],:]   for r in the tile's producer range -> LDS
//            (+ HBM for the rows the remainder will read)
//   phase 2  D[i,:] = sum_k Ax[k] * T[Ai[k],:]   for the tile's fused rows, T read from LDS
// ---------------------------------------------------------------------------------
template <int V, int LPR>
__global__ __launch_bounds__(kBlock) void fused_spmm_spmm_kernel(
    const TileDesc *__restrict__ tiles, int n_tiles, int per_xcd, const int *__restrict__ fused_ids,
    const int *__restrict__ Bp, const int *__restrict__ Bi, const float *__restrict__ Bx,
    const float *__restrict__ C, const int *__restrict__ Ap, const int *__restrict__ Ai,
    const float *__restrict__ Ax, float *__restrict__ D, float *__restrict__ T, int N, int ldc,
    int accumulate) {
  extern __shared__ __align__(16) float slab[];
  const int tile = xcd_contiguous(blockIdx.x, per_xcd);
  if (tile >= n_tiles) return;
  const TileDesc t = tiles[tile];
  constexpr int G = kBlock / LPR;
  const int group = threadIdx.x / LPR, glane = threadIdx.x % LPR;
  const bool has_cons = t.cons_end > t.cons_begin;
  for (int c0 = 0; c0 < N; c0 += LPR * V) {
    const int coff = c0 + glane * V;
    const bool ok = coff < N;
    const GlobalRows<V> csrc{C, ldc, ok ? coff : 0};
    for (int r = t.prod_begin + group; r < t.prod_end; r += G) {
      fvec<V> acc = vzero<V>();
      row_dot<V, LPR>(Bi, Bx, Bp[r], Bp[r + 1], glane, ok, csrc, acc);
      if (ok) {
        if (has_cons) *reinterpret_cast<fvec<V> *>(slab + (r - t.prod_begin) * N + coff) = acc;
        if (r >= t.wb_begin && r < t.wb_end)
          *reinterpret_cast<fvec<V> *>(T + (size_t)r * N + coff) = acc;
      }
    }
    if (!has_cons) continue;
    __syncthreads();
    const LdsRows<V> tsrc{slab, N, ok ? coff : 0, t.prod_begin};
    for (int q = t.cons_begin + group; q < t.cons_end; q += G) {
      const int i = fused_ids[q];
      fvec<V> acc = vzero<V>();
      if (accumulate && ok) acc = *reinterpret_cast<const fvec<V> *>(D + (size_t)i * N + coff);
      row_dot<V, LPR>(Ai, Ax, Ap[i], Ap[i + 1], glane, ok, tsrc, acc);
      if (ok) store_streaming<V>(D + (size_t)i * N + coff, acc);
    }
  }
}

// ---------------------------------------------------------------------------------
// Windowed fused SpMM-SpMM tile kernel (inner matrix == outer matrix, the reference's
// setting).  Everything a tile touches more than once is staged in LDS first:
//   * the CSR chunk of its producer rows, as (byte offset into the window, value) pairs,
//     one pad entry per row so that the rows a wavefront walks start in different banks;
//   * then, strip by strip (SW columns of C/D at a time): the window of C rows the
//     producer rows read, the slab of intermediate rows, and out of it the fused rows.
// A lane group of SW/4 lanes owns one row; both products read only LDS, HBM sees each
// C row about once per tile and each D row once.  Same fma sequence per element as
// fused_spmm_spmm_kernel, hence the same bits.
// ---------------------------------------------------------------------------------
constexpr int kWinPad = 2;  // pad slots after each staged row (keeps 8 rows' reads in 8 bank groups)

__device__ __forceinline__ int align16i(int x) { return (x + 15) & ~15; }

// acc += sum_k val[k] * row(off[k]) over staged entries [kb, ke), in order.  The entry
// reads of the next four are issued before the fmas of the current four.
__device__ __forceinline__ fvec<4> lds_row_dot(const int2 *__restrict__ ent, int kb, int ke,
                                               const char *base, fvec<4> acc) {
  int k = kb;
  if (k + 4 <= ke) {
    int2 e0 = ent[k], e1 = ent[k + 1], e2 = ent[k + 2], e3 = ent[k + 3];
    k += 4;
    for (;;) {
      const fvec<4> x0 = *reinterpret_cast<const fvec<4> *>(base + e0.x);
      const fvec<4> x1 = *reinterpret_cast<const fvec<4> *>(base + e1.x);
      const fvec<4> x2 = *reinterpret_cast<const fvec<4> *>(base + e2.x);
      const fvec<4> x3 = *reinterpret_cast<const fvec<4> *>(base + e3.x);
      const bool more = k + 4 <= ke;
      int2 n0 = e0, n1 = e1, n2 = e2, n3 = e3;
      if (more) { n0 = ent[k]; n1 = ent[k + 1]; n2 = ent[k + 2]; n3 = ent[k + 3]; }
      vfma<4>(__int_as_float(e0.y), x0, acc);
      vfma<4>(__int_as_float(e1.y), x1, acc);
      vfma<4>(__int_as_float(e2.y), x2, acc);
      vfma<4>(__int_as_float(e3.y), x3, acc);
      if (!more) break;
      e0 = n0; e1 = n1; e2 = n2; e3 = n3;
      k += 4;
    }
  }
  for (; k < ke; ++k) {
    const int2 e0 = ent[k];
    vfma<4>(__int_as_float(e0.y), *reinterpret_cast<const fvec<4> *>(base + e0.x), acc);
  }
  return acc;
}

// The value lane G of the caller's quad holds (a DPP quad_perm broadcast, folded into the
// consuming instruction: no LDS traffic and no instruction of its own).
template <int G> __device__ __forceinline__ int quad_bcast(int v) {
  return __builtin_amdgcn_mov_dpp(v, G * 0x55, 0xf, 0xf, true);
}

// acc += (val as held by lane G of the quad) * x: four v_fmac_f32 with the DPP broadcast on the
// value operand.  (Written out because the compiler folds a broadcast into its consumer only
// when there is a single one.  The value register is filled by a load; the two idle cycles
// cover the case of a register copy placed right in front, which a DPP read must not follow
// directly.)
template <int G> __device__ __forceinline__ void quad_fma(int val, const fvec<4> &x, fvec<4> &acc) {
  asm("s_nop 1\n\t"
      "v_fmac_f32_dpp %0, %4, %5 quad_perm:[%9,%9,%9,%9] row_mask:0xf bank_mask:0xf bound_ctrl:0\n\t"
      "v_fmac_f32_dpp %1, %4, %6 quad_perm:[%9,%9,%9,%9] row_mask:0xf bank_mask:0xf bound_ctrl:0\n\t"
      "v_fmac_f32_dpp %2, %4, %7 quad_perm:[%9,%9,%9,%9] row_mask:0xf bank_mask:0xf bound_ctrl:0\n\t"
      "v_fmac_f32_dpp %3, %4, %8 quad_perm:[%9,%9,%9,%9] row_mask:0xf bank_mask:0xf bound_ctrl:0"
      : "+v"(acc.v[0]), "+v"(acc.v[1]), "+v"(acc.v[2]), "+v"(acc.v[3])
      : "v"(val), "v"(x.v[0]), "v"(x.v[1]), "v"(x.v[2]), "v"(x.v[3]), "n"(G));
}

// Eight staged entries, held four to a lane by lanes GA and GB of the quad: gathers first, then the fmas in order.
template <int GA, int GB, bool CHECK>
__device__ __forceinline__ void quad_dot8(const int2 (&e)[4], const char *base, int left, fvec<4> &acc) {
  fvec<4> x[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (!CHECK || 4 * GA + j < left) x[j] = *reinterpret_cast<const fvec<4> *>(base + quad_bcast<GA>(e[j].x));
    if (!CHECK || 4 * GB + j < left) x[4 + j] = *reinterpret_cast<const fvec<4> *>(base + quad_bcast<GB>(e[j].x));
  }
#pragma unroll
  for (int j = 0; j < 4; ++j)
    if (!CHECK || 4 * GA + j < left) quad_fma<GA>(e[j].y, x[j], acc);
#pragma unroll
  for (int j = 0; j < 4; ++j)
    if (!CHECK || 4 * GB + j < left) quad_fma<GB>(e[j].y, x[4 + j], acc);
}

// acc += sum_k val[k] * row(off[k]) over staged entries [kb, ke), in order, for a lane group
// that is a whole number of quads.  A lane reads only every fourth run of four entries
// (q = its position in its quad says which); the other twelve of each sixteen come from its
// quad's lanes through DPP.  Against lds_row_dot this trades one LDS read of 8 bytes per lane
// and entry for one of 32 bytes per lane and sixteen entries.
__device__ __forceinline__ fvec<4> lds_row_dot_quad(const int2 *__restrict__ ent, int kb, int ke, const char *base,
                                                    int q, fvec<4> acc) {
  for (int c = kb; c < ke; c += 16) {
    const int2 *p = ent + c + 4 * q;  // (may run past the row's end: those entries are not used)
    const int2 e[4] = {p[0], p[1], p[2], p[3]};
    const int left = ke - c;
    if (left >= 16) {
      quad_dot8<0, 1, false>(e, base, left, acc);
      quad_dot8<2, 3, false>(e, base, left, acc);
    } else {
      quad_dot8<0, 1, true>(e, base, left, acc);
      if (left > 8) quad_dot8<2, 3, true>(e, base, left, acc);
    }
  }
  return acc;
}

// One 16-byte unit of a strip of the window of C (unit u = row-in-window * LPR + quad).
// Threads past the end re-read unit 0, which always exists; the value is not used.
template <int LPR>
__device__ __forceinline__ fvec<4> window_unit(const float *__restrict__ C, int first_row, int N, int c0,
                                               int n4, int u) {
  const int uu = u < n4 ? u : 0;
  return load_streaming4(C + (size_t)(first_row + uu / LPR) * N + c0 + (uu % LPR) * 4);
}

template <int SW, int BLOCK, bool ACC>
__global__ __launch_bounds__(BLOCK) void fused_spmm_spmm_window_kernel(
    const TileDesc *__restrict__ tiles, const int2 *__restrict__ win, int n_tiles, int per_xcd,
    const int *__restrict__ fused_ids, const int *__restrict__ Bp, const int *__restrict__ Bi,
    const float *__restrict__ Bx, const float *__restrict__ C, float *__restrict__ D, int N) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int LPR = SW / 4;           // lanes per row
  constexpr int G = BLOCK / LPR;        // rows in flight per workgroup
  constexpr int ROWB = SW * 4;          // bytes of one strip row
  const int tile = xcd_contiguous(blockIdx.x, per_xcd);
  if (tile >= n_tiles) return;
  const TileDesc t = tiles[tile];
  const int2 w = win[tile];
  const int P = t.prod_end - t.prod_begin, R = t.cons_end - t.cons_begin, Wc = w.y - w.x;
  const int k0 = Bp[t.prod_begin];
  const int nz = Bp[t.prod_end] - k0;
  int *rp = reinterpret_cast<int *>(smem);
  int *cons = reinterpret_cast<int *>(smem + align16i(4 * (P + 1)));
  int2 *ent = reinterpret_cast<int2 *>(reinterpret_cast<unsigned char *>(cons) + align16i(4 * R));
  float *Cbuf = reinterpret_cast<float *>(reinterpret_cast<unsigned char *>(ent) + align16i(8 * (nz + kWinPad * P)));
  float *Tbuf = Cbuf + Wc * SW;
  const int tid = threadIdx.x, group = tid / LPR, glane = tid % LPR;

  const int n4 = Wc * LPR;  // 16-byte units in one strip of the window
  // The next strip of the window is fetched into registers while the current one is being
  // worked on, and dropped into LDS once the current strip's first product is done.
  constexpr int UPT = 4;  // register-prefetched 16-byte units per thread
  fvec<4> pre0 = window_unit<LPR>(C, w.x, N, 0, n4, tid);
  fvec<4> pre1 = window_unit<LPR>(C, w.x, N, 0, n4, tid + BLOCK);
  fvec<4> pre2 = window_unit<LPR>(C, w.x, N, 0, n4, tid + 2 * BLOCK);
  fvec<4> pre3 = window_unit<LPR>(C, w.x, N, 0, n4, tid + 3 * BLOCK);
  // row pointers: entry j of row i sits at rp[i] + j, kWinPad unused slots follow every row
  for (int i = tid; i <= P; i += BLOCK) rp[i] = Bp[t.prod_begin + i] - k0 + kWinPad * i;
  for (int i = tid; i < R; i += BLOCK) cons[i] = fused_ids[t.cons_begin + i] - t.prod_begin;
  // entries: one lane group per row
  for (int r = group; r < P; r += G) {
    const int kb = Bp[t.prod_begin + r], ke = Bp[t.prod_begin + r + 1];
    const int dst = kb - k0 + kWinPad * r;
    for (int k = kb + glane; k < ke; k += LPR)
      ent[dst + (k - kb)] = make_int2((Bi[k] - w.x) * ROWB, __float_as_int(Bx[k]));
  }
  const char *cbase = reinterpret_cast<const char *>(Cbuf) + glane * 16;
  // a consumer's column c lives in the slab at row c - prod_begin = (c - w.x) + (w.x - prod_begin)
  const char *tbase = reinterpret_cast<const char *>(Tbuf) + (w.x - t.prod_begin) * ROWB + glane * 16;
  for (int c0 = 0; c0 < N; c0 += SW) {
    __syncthreads();  // previous strip fully consumed (and, first time, staging visible)
    {
      fvec<4> *cb = reinterpret_cast<fvec<4> *>(Cbuf);
      if (tid < n4) cb[tid] = pre0;
      if (tid + BLOCK < n4) cb[tid + BLOCK] = pre1;
      if (tid + 2 * BLOCK < n4) cb[tid + 2 * BLOCK] = pre2;
      if (tid + 3 * BLOCK < n4) cb[tid + 3 * BLOCK] = pre3;
      for (int u = tid + UPT * BLOCK; u < n4; u += BLOCK)  // windows beyond the prefetch capacity
        cb[u] = window_unit<LPR>(C, w.x, N, c0, n4, u);
    }
    if (c0 + SW < N) {
      pre0 = window_unit<LPR>(C, w.x, N, c0 + SW, n4, tid);
      pre1 = window_unit<LPR>(C, w.x, N, c0 + SW, n4, tid + BLOCK);
      pre2 = window_unit<LPR>(C, w.x, N, c0 + SW, n4, tid + 2 * BLOCK);
      pre3 = window_unit<LPR>(C, w.x, N, c0 + SW, n4, tid + 3 * BLOCK);
    }
    __syncthreads();
    for (int r = group; r < P; r += G) {
      const fvec<4> acc = lds_row_dot_quad(ent, rp[r], rp[r + 1] - kWinPad, cbase, glane & 3, vzero<4>());
      *reinterpret_cast<fvec<4> *>(Tbuf + r * SW + glane * 4) = acc;
    }
    __syncthreads();
    for (int q = group; q < R; q += G) {
      const int r = cons[q];
      float *dst = D + (size_t)(t.prod_begin + r) * N + c0 + glane * 4;
      fvec<4> acc = vzero<4>();
      // (a compile-time switch: a load under a run-time condition would make every store of
      // this loop wait for the one before it)
      if constexpr (ACC) acc = *reinterpret_cast<const fvec<4> *>(dst);
      acc = lds_row_dot_quad(ent, rp[r], rp[r + 1] - kWinPad, tbase, glane & 3, acc);
      store_streaming<4>(dst, acc);
    }
  }
}

// ---------------------------------------------------------------------------------
// Windowed fused SpMM-SpMM tile kernel for long matrices: strips of 64 columns, one
// workgroup of 1024 threads (and up to the whole LDS) per compute unit.  The LDS of this GPU
// reads 256 bytes a clock when the 16 lanes it serves together touch 64 different banks; a
// 256-byte strip row read by a 16-lane group does, two 128-byte rows read by two 8-lane groups
// collide whenever the rows sit on the same half of the banks (every second pair of rows).
// The price is a row twice as large, so the tile's entries are not staged in LDS: a lane
// loads its four of every sixteen from the CSR arrays (the rest reach it through its quad),
// one row ahead of the row it works on.  Same fma sequence per element as the kernels above.
// ---------------------------------------------------------------------------------
constexpr int kW64Strip = 64, kW64Block = 1024;
typedef int int4u __attribute__((ext_vector_type(4), aligned(4)));
typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));

struct QuadEntries {  // entries [k, k + 4) of a row as (byte offset into the window, value bits)
  int2 e[4];
  int kb, ke;  // the row's entry range (kept by the row loops next to the entries fetched ahead)
};

// Entries k .. k+3 of the CSR arrays as (byte offset into the window, value bits); off0 is
// minus the window's first column times the row size.  EXACT: the caller may be within four
// entries of the end of the arrays (the last tile of the matrix), so a lane that would read
// past them loads one entry at a time; elsewhere the four come as one load each.
template <bool EXACT>
__device__ __forceinline__ QuadEntries load_quad_entries(const int *__restrict__ ci, const float *__restrict__ cv, int k,
                                                         int end_k, int nnz, int off0) {
  QuadEntries r;
  const int kk = EXACT ? min(k, nnz - 4) : k;  // (nnz >= 4: checked on the host)
  const unsigned byte = (unsigned)kk * 4u;    // (one 32-bit offset from both array bases)
  const int4u c = *reinterpret_cast<const int4u *>(reinterpret_cast<const char *>(ci) + byte);
  const float4u v = *reinterpret_cast<const float4u *>(reinterpret_cast<const char *>(cv) + byte);
#pragma unroll
  for (int j = 0; j < 4; ++j) r.e[j] = make_int2((c[j] << 8) + off0, __float_as_int(v[j]));
  if constexpr (EXACT) {
    if (kk != k && k < end_k) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int kj = min(k + j, nnz - 1);
        r.e[j] = make_int2((ci[kj] << 8) + off0, __float_as_int(cv[kj]));
      }
    }
  }
  return r;
}
static_assert(kW64Strip * 4 == 1 << 8, "row size of the 64-column strip");

// acc += the row's entries [kb, ke) times their window rows; `first` holds this lane's four of
// the first sixteen.
template <bool EXACT>
__device__ __forceinline__ fvec<4> row_dot_quad_regs(const QuadEntries &first, const int *__restrict__ ci,
                                                     const float *__restrict__ cv, int kb, int ke, int nnz,
                                                     int off0, const char *base, int q, fvec<4> acc) {
  const int n = ke - kb;
  if (n >= 16) {
    quad_dot8<0, 1, false>(first.e, base, n, acc);
    quad_dot8<2, 3, false>(first.e, base, n, acc);
  } else {
    quad_dot8<0, 1, true>(first.e, base, n, acc);
    if (n > 8) quad_dot8<2, 3, true>(first.e, base, n, acc);
  }
  for (int c = kb + 16; c < ke; c += 16) {
    const QuadEntries cur = load_quad_entries<EXACT>(ci, cv, c + 4 * q, ke, nnz, off0);
    const int left = ke - c;
    if (left >= 16) {
      quad_dot8<0, 1, false>(cur.e, base, left, acc);
      quad_dot8<2, 3, false>(cur.e, base, left, acc);
    } else {
      quad_dot8<0, 1, true>(cur.e, base, left, acc);
      if (left > 8) quad_dot8<2, 3, true>(cur.e, base, left, acc);
    }
  }
  return acc;
}

template <bool ACC>
__global__ __launch_bounds__(kW64Block) void fused_spmm_spmm_window64_kernel(
    const TileDesc *__restrict__ tiles, const int2 *__restrict__ win, int n_tiles, int per_xcd,
    const int *__restrict__ Bp, const int *__restrict__ Bi, const float *__restrict__ Bx, int nnzB,
    const float *__restrict__ C, const int *__restrict__ Ap, const int *__restrict__ Ai,
    const float *__restrict__ Ax, int nnzA, float *__restrict__ D, int N, int n_loaders) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int SW = kW64Strip, LPR = SW / 4, G = kW64Block / LPR, ROWB = SW * 4;
  const int tile = xcd_contiguous(blockIdx.x, per_xcd);
  if (tile >= n_tiles) return;
  const TileDesc t = tiles[tile];
  const int2 w = win[tile];
  // (a windowed tile's fused rows are its own rows, in order)
  const int P = t.prod_end - t.prod_begin, R = t.cons_end - t.cons_begin, Wc = w.y - w.x;
  int *rpB = reinterpret_cast<int *>(smem);                        // row pointers of the producer rows (B)
  int *rpA = reinterpret_cast<int *>(smem + align16i(4 * (P + 1)));  // ... and of the fused rows (A)
  float *Cbuf = reinterpret_cast<float *>(reinterpret_cast<unsigned char *>(rpA) + align16i(4 * (R + 1)));
  float *Tbuf = Cbuf + Wc * SW;
  const int tid = threadIdx.x, group = tid / LPR, glane = tid % LPR, q = glane & 3;
  const int n4 = Wc * LPR;
  // The window of C goes from global memory straight into LDS (no registers): one instruction of
  // a wavefront moves 64 units of 16 bytes, i.e. four window rows, to consecutive LDS addresses.
  const int wave = tid / 64, lane = tid % 64;
  auto stage_window = [&](int c0, int first_wave, int n_waves) {
    for (int u0 = (wave - first_wave) * 64; u0 < n4; u0 += n_waves * 64) {
      const int u = u0 + lane;
      if (u < n4)
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void *)(C + (size_t)(w.x + u / 16) * N + c0 + (u % 16) * 4),
            (__attribute__((address_space(3))) void *)(Cbuf + u0 * 4), 16, 0, 0);
    }
  };
  stage_window(0, 0, kW64Block / 64);
  for (int i = tid; i <= P; i += kW64Block) rpB[i] = Bp[t.prod_begin + i];
  for (int i = tid; i <= R; i += kW64Block) rpA[i] = Ap[t.own_begin + i];
  // column c of B is row c - w.x of the window, column c of A row c - prod_begin of the slab
  const char *cbase = reinterpret_cast<const char *>(Cbuf) + glane * 16;
  const char *tbase = reinterpret_cast<const char *>(Tbuf) + glane * 16;
  const int offB = -w.x * ROWB, offA = -t.prod_begin * ROWB;
  // (only the last tile of the matrix can come within a load of the end of the arrays)
  const bool near_end = Bp[t.prod_end] + 16 > nnzB || Ap[t.own_begin + R] + 16 > nnzA;
  auto products = [&](auto exact_tag, int c0) {
    const bool more = c0 + SW < N;  // another strip follows: its window is fetched during the second product
    constexpr bool EXACT = decltype(exact_tag)::value;
    QuadEntries ea, eb;
    auto fetchB = [&](int r) {
      const int rr = min(r, P - 1);
      const int kb = rpB[rr], ke = rpB[rr + 1];
      QuadEntries e = load_quad_entries<EXACT>(Bi, Bx, kb + 4 * q, ke, nnzB, offB);
      e.kb = kb; e.ke = ke;
      return e;
    };
    auto fetchA = [&](int r) {
      const int rr = min(r, R - 1);
      const int kb = rpA[rr], ke = rpA[rr + 1];
      QuadEntries e = load_quad_entries<EXACT>(Ai, Ax, kb + 4 * q, ke, nnzA, offA);
      e.kb = kb; e.ke = ke;
      return e;
    };
    // first product: slab rows 0 .. P-1, a lane group per row, the next row's entries on their way
    ea = fetchB(group);
    for (int r = group; r < P; r += 2 * G) {
      eb = fetchB(r + G);
      *reinterpret_cast<fvec<4> *>(Tbuf + r * SW + glane * 4) =
          row_dot_quad_regs<EXACT>(ea, Bi, Bx, ea.kb, ea.ke, nnzB, offB, cbase, q, vzero<4>());
      if (r + G >= P) break;
      ea = fetchB(r + 2 * G);
      *reinterpret_cast<fvec<4> *>(Tbuf + (r + G) * SW + glane * 4) =
          row_dot_quad_regs<EXACT>(eb, Bi, Bx, eb.kb, eb.ke, nnzB, offB, cbase, q, vzero<4>());
    }
    lds_barrier();
    // then the fused rows out of the slab.  The window is free now: while another strip follows,
    // the last n_loaders wavefronts fetch its window instead of taking rows (their loads would
    // otherwise stand in front of every entry load of this product: loads return in order).
    const int g2 = more ? G - n_loaders * (64 / LPR) : G;
    if (more && group >= g2) {
      stage_window(c0 + SW, kW64Block / 64 - n_loaders, n_loaders);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else {
      if (R > 0) ea = fetchA(group);
      float *dst = D + (size_t)(t.own_begin + group) * N + c0 + glane * 4;
      const size_t round_stride = (size_t)g2 * N;
      for (int i = group; i < R; i += 2 * g2) {
        eb = fetchA(i + g2);
        {
          fvec<4> acc = vzero<4>();
          if constexpr (ACC) acc = *reinterpret_cast<const fvec<4> *>(dst);
          store_streaming<4>(dst, row_dot_quad_regs<EXACT>(ea, Ai, Ax, ea.kb, ea.ke, nnzA, offA, tbase, q, acc));
          dst += round_stride;
        }
        if (i + g2 >= R) break;
        ea = fetchA(i + 2 * g2);
        {
          fvec<4> acc = vzero<4>();
          if constexpr (ACC) acc = *reinterpret_cast<const fvec<4> *>(dst);
          store_streaming<4>(dst, row_dot_quad_regs<EXACT>(eb, Ai, Ax, eb.kb, eb.ke, nnzA, offA, tbase, q, acc));
          dst += round_stride;
        }
      }
    }
    lds_barrier();  // slab consumed, next window (if any) in LDS
  };
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's part of the first window has landed
  lds_barrier();                                    // ... and everybody's, and the row pointers
  for (int c0 = 0; c0 < N; c0 += SW) {
    if (near_end) products(std::true_type{}, c0);
    else products(std::false_type{}, c0);
  }
}

// ---------------------------------------------------------------------------------
// Row-wise SpMM  Y[i,:] = sum_k Ax[k] * X[Ai[k],:]  for i = rows[q] (or i = q when rows
// is null).  Serves the unfused remainder (X = the intermediate in HBM), producer rows
// that no tile fuses, and tf_spmm.  One lane group per row and small, short-lived
// workgroups: what hides the gather latency is the number of rows in flight.
// ---------------------------------------------------------------------------------
template <int V, int LPR, bool COAL, bool FLAG = false>
__global__ __launch_bounds__(kBlock) void spmm_rows_kernel(
    const int *__restrict__ rows, int n_rows, int n_blocks, int per_xcd, const int *__restrict__ Ap,
    const int *__restrict__ Ai, const float *__restrict__ Ax, const float *__restrict__ X, int ldx,
    float *__restrict__ Y, int N, int accumulate, int streaming, int compact) {
  constexpr int G = kBlock / LPR;
  const int group = threadIdx.x / LPR, glane = threadIdx.x % LPR;
  const int b = xcd_contiguous(blockIdx.x, per_xcd);
  if (b >= n_blocks) return;
  const int q = b * G + group;
  if (q >= n_rows) return;  // whole lane groups leave together
  const int i = rows ? rows[q] : q;
  // compact: the CSR arrays hold the listed rows only, in the order of the list (the reference's
  // reordered adjacency: consumer rows stored in schedule order), so row q of them is row rows[q] of Y
  const int r = compact ? q : i;
  const int kb = Ap[r], ke = Ap[r + 1];
  for (int c0 = 0; c0 < N; c0 += LPR * V) {
    const int coff = c0 + glane * V;
    const bool ok = coff < N;
    const GlobalRows<V> src{X, ldx, ok ? coff : 0};
    fvec<V> acc = vzero<V>();
    if (accumulate && ok) acc = *reinterpret_cast<const fvec<V> *>(Y + (size_t)i * N + coff);
    // COAL: the group's lanes load the pairs of up to LPR entries with one coalesced request and hand
    // them round by shuffles -- one round trip for the pairs of a long row or segment instead of one
    // per eight entries (hot long-row segments of the R-MAT step, 22 entries on average: 0.86 -> 0.74
    // ms).  Rows of a few entries, and segments whose gathers all miss L2, are served as well or
    // better by every lane reading the pairs itself (cold segments 0.27 -> 0.29 ms).
    // FLAG: column indices carry the schedule's "cold" mark in their top bit (see GlobalRows::load_flagged)
    if constexpr (COAL) row_dot<V, LPR, GlobalRows<V>, FLAG>(Ai, Ax, kb, ke, glane, ok, src, acc);
    else row_dot_direct<V, LPR, GlobalRows<V>, FLAG>(Ai, Ax, kb, ke, ok, src, acc);
    if (ok) {
      if (streaming) store_streaming<V>(Y + (size_t)i * N + coff, acc);
      else *reinterpret_cast<fvec<V> *>(Y + (size_t)i * N + coff) = acc;
    }
  }
}

// ---------------------------------------------------------------------------------
// Long remainder rows.  One workgroup per chunk of a row: lane groups take LPR-entry
// segments round-robin, partial sums are combined across the groups through LDS in a
// fixed order, and the chunk's result goes to partial[slot].  A second kernel adds a
// row's chunks in order, so the result does not depend on scheduling.
// ---------------------------------------------------------------------------------
template <int V, int LPR>
__global__ __launch_bounds__(kBlock) void spmm_long_chunk_kernel(
    const LongChunk *__restrict__ chunks, const int *__restrict__ Ai, const float *__restrict__ Ax,
    const float *__restrict__ X, int ldx, float *__restrict__ partial, int N) {
  constexpr int G = kBlock / LPR;
  __shared__ __align__(16) float red[G * LPR * V];
  const LongChunk ch = chunks[blockIdx.x];
  const int group = threadIdx.x / LPR, glane = threadIdx.x % LPR;
  for (int c0 = 0; c0 < N; c0 += LPR * V) {
    const int coff = c0 + glane * V;
    const bool ok = coff < N;
    const GlobalRows<V> src{X, ldx, ok ? coff : 0};
    fvec<V> acc = vzero<V>();
    for (int k0 = ch.k_begin + group * LPR; k0 < ch.k_end; k0 += G * LPR)
      row_dot<V, LPR>(Ai, Ax, k0, min(ch.k_end, k0 + LPR), glane, ok, src, acc);
    *reinterpret_cast<fvec<V> *>(red + (group * LPR + glane) * V) = acc;
    __syncthreads();
    if (group == 0 && ok) {
      fvec<V> sum = vzero<V>();
      for (int g = 0; g < G; ++g) vadd<V>(*reinterpret_cast<const fvec<V> *>(red + (g * LPR + glane) * V), sum);
      *reinterpret_cast<fvec<V> *>(partial + (size_t)ch.slot * N + coff) = sum;
    }
    __syncthreads();
  }
}

__global__ __launch_bounds__(kBlock) void long_row_reduce_kernel(const LongRow *__restrict__ rows,
                                                                 const float *__restrict__ partial,
                                                                 float *__restrict__ Y, int N,
                                                                 int accumulate) {
  const LongRow lr = rows[blockIdx.x];
  for (int c = threadIdx.x; c < N; c += kBlock) {
    float s = accumulate ? Y[(size_t)lr.row * N + c] : 0.f;
    for (int p = 0; p < lr.count; ++p) s += partial[(size_t)(lr.first + p) * N + c];
    Y[(size_t)lr.row * N + c] = s;
  }
}

// out[i] = val[src[i]]: the values of the rows of a list, in the order of the list.
__global__ void gather_values_kernel(const int *__restrict__ src, const float *__restrict__ val, float *__restrict__ out, int n) {
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) out[i] = val[src[i]];
}

// Column-partitioned long rows: out[pos[i]] = val[src[i]] puts the values of A into the order of
// the regrouped entries (src ascending: the reads walk A's array once, the writes fall into
// nine ascending streams), and Y[row] (+)= the row's segment sums, added in the order of its list.
__global__ void scatter_values_kernel(const int *__restrict__ src, const int *__restrict__ pos,
                                      const float *__restrict__ val, float *__restrict__ out, int n) {
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) out[pos[i]] = val[src[i]];
}

// One lane group per long row, every lane four adjacent columns; the partial rows of eight
// segments are requested before the first is added.
template <int V, int LPR>
__global__ __launch_bounds__(kBlock) void long_seg_reduce_kernel(const LongRow *__restrict__ rows, int n_long,
                                                                 const int *__restrict__ seg_of,
                                                                 const float *partial, float *Y, int N,
                                                                 int accumulate) {  // (Y may be `partial` itself: other rows)
  constexpr int G = kBlock / LPR;
  const int group = threadIdx.x / LPR, glane = threadIdx.x % LPR;
  const int q = blockIdx.x * G + group;
  if (q >= n_long) return;
  const LongRow lr = rows[q];
  for (int c0 = 0; c0 < N; c0 += LPR * V) {
    const int coff = c0 + glane * V;
    if (coff >= N) continue;
    fvec<V> acc = vzero<V>();
    if (accumulate) acc = *reinterpret_cast<const fvec<V> *>(Y + (size_t)lr.row * N + coff);
    for (int p0 = 0; p0 < lr.count; p0 += 8) {
      fvec<V> x[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (p0 + u < lr.count) x[u] = *reinterpret_cast<const fvec<V> *>(partial + (size_t)seg_of[lr.first + p0 + u] * N + coff);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (p0 + u < lr.count) vadd<V>(x[u], acc);
    }
    *reinterpret_cast<fvec<V> *>(Y + (size_t)lr.row * N + coff) = acc;
  }
}

// dst (rows x ld_dst) = src (src_rows x ld_src) in its top left corner, zeros elsewhere.
__global__ void pad_kernel(const float *__restrict__ src, int src_rows, int ld_src, float *__restrict__ dst, int rows,
                           int ld_dst) {
  const size_t n = (size_t)rows * ld_dst;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const int r = (int)(i / ld_dst), c = (int)(i % ld_dst);
    dst[i] = (r < src_rows && c < ld_src) ? src[(size_t)r * ld_src + c] : 0.f;
  }
}

// dst[r, dst_col0 + c] (+)= src[r, src_col0 + c] for r < rows, c < cols; zero where src has no such row or column
// (rows >= src_rows, c >= src_cols).  Column panels of C and D when N is not a width the MFMA kernels take.
__global__ void copy_cols_kernel(const float *__restrict__ src, int src_rows, int ld_src, int src_col0, int src_cols,
                                 float *__restrict__ dst, int rows, int ld_dst, int dst_col0, int cols, int accumulate) {
  const size_t n = (size_t)rows * cols;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const int r = (int)(i / cols), c = (int)(i % cols);
    const float v = (r < src_rows && c < src_cols) ? src[(size_t)r * ld_src + src_col0 + c] : 0.f;
    float *p = dst + (size_t)r * ld_dst + dst_col0 + c;
    *p = accumulate ? *p + v : v;
  }
}

// Rows of zeros: Y[rows[q], :] = 0 (second-op rows without entries), V floats per thread.
template <int V>
__global__ void zero_rows_kernel(const int *__restrict__ rows, size_t units, float *__restrict__ Y, int N) {
  const int per_row = N / V;
  for (size_t u = blockIdx.x * (size_t)blockDim.x + threadIdx.x; u < units; u += (size_t)gridDim.x * blockDim.x) {
    const size_t q = u / per_row;
    const int c = (int)(u - q * per_row) * V;
    store_streaming<V>(Y + (size_t)rows[q] * N + c, vzero<V>());  // (plain stores: this launch 5 % faster, the next one 5 % slower)
  }
}

// p = max(p, 0) over n values: four per thread, and the up to three values behind the last four one each.
__global__ void relu_kernel(float *__restrict__ p, size_t n) {
  const size_t n4 = n / 4;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n4; i += (size_t)gridDim.x * blockDim.x) {
    fvec<4> v = *reinterpret_cast<const fvec<4> *>(p + 4 * i);
#pragma unroll
    for (int c = 0; c < 4; ++c) v.v[c] = fmaxf(v.v[c], 0.f);
    *reinterpret_cast<fvec<4> *>(p + 4 * i) = v;
  }
  if (blockIdx.x == 0 && 4 * n4 + threadIdx.x < n) p[4 * n4 + threadIdx.x] = fmaxf(p[4 * n4 + threadIdx.x], 0.f);
}

// out[workgroup] = the XCD it runs on (hardware register XCC_ID, bits 3:0).
__global__ void xcd_probe_kernel(int *__restrict__ out) {
  if (threadIdx.x == 0) out[blockIdx.x] = (int)__builtin_amdgcn_s_getreg(20 | (0 << 6) | ((4 - 1) << 11));
}

__global__ void fill_kernel(float *__restrict__ p, size_t n, float v) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}

// ---------------------------------------------------------------------------------
// Tile GEMM on fp32 MFMA.  A wavefront owns a block of 32 rows and all N = 32*NB
// columns: NB accumulators of v_mfma_f32_32x32x2_f32.  C (K x N) is staged through LDS
// kc rows at a time; the rows of B are read straight from HBM, 16 bytes per lane: lane
// (i = lane%32, h = lane/32) loads B[row0+i][k0+8m+4h .. +4), so one load feeds four
// MFMA steps whose k index is 8m+4h+t.  The same k is used for the C operand, so the
// permuted k order inside a group of 8 does not change the product.
// ---------------------------------------------------------------------------------
typedef float v16f __attribute__((ext_vector_type(16)));

template <int NB>
__device__ __forceinline__ void gemm_accumulate_chunk(const float *__restrict__ Xrow, bool row_ok,
                                                      int kc, const float *stage, int N, int h, int j,
                                                      v16f (&acc)[NB]) {
  for (int m = 0; m < kc; m += 8) {
    fvec<4> a4 = vzero<4>();
    if (row_ok) a4 = *reinterpret_cast<const fvec<4> *>(Xrow + m + 4 * h);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float *w = stage + (m + 4 * h + t) * N + j;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        acc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4.v[t], w[nb * 32], acc[nb], 0, 0, 0);
    }
  }
}

// Cooperative copy of rows [k0, k0+kc) of W (K x N, row-major) into LDS.
__device__ __forceinline__ void stage_weights(const float *__restrict__ W, int N, int k0, int kc, float *stage) {
  const int n4 = kc * N / 4;
  const fvec<4> *src = reinterpret_cast<const fvec<4> *>(W + (size_t)k0 * N);
  fvec<4> *dst = reinterpret_cast<fvec<4> *>(stage);
  for (int i = threadIdx.x; i < n4; i += kBlock) dst[i] = src[i];
}

// Computes intermediate rows [p0, p1) = X[p0:p1, :K] * W for the whole workgroup.
// Results go to `slab` (row r at (r-p0)*N) when slab != null and to T rows in
// [wb0, wb1) when T != null.  Must be called by all threads of the workgroup.
template <int NB>
__device__ __forceinline__ void tile_gemm(const float *__restrict__ X, const float *__restrict__ W, int K,
                                          int kc, int p0, int p1, float *stage, float *slab,
                                          float *__restrict__ T, int wb0, int wb1) {
  constexpr int N = NB * 32;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int h = lane / 32, j = lane % 32;
  constexpr int W_PER_BLOCK = kBlock / 64;
  const int nrb = (p1 - p0 + 31) / 32;
  const int iters = (nrb + W_PER_BLOCK - 1) / W_PER_BLOCK;
  const bool single = (K <= kc);
  if (single) {
    stage_weights(W, N, 0, K, stage);
    __syncthreads();
  }
  for (int it = 0; it < iters; ++it) {
    const int rb = it * W_PER_BLOCK + wave;
    const int row = p0 + rb * 32 + j;  // the row this lane feeds as the A operand
    const bool row_ok = rb < nrb && row < p1;
    const float *Xrow = X + (size_t)(row_ok ? row : p0) * K;
    v16f acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[nb][r] = 0.f;
    if (single) {
      if (rb < nrb) gemm_accumulate_chunk<NB>(Xrow, row_ok, K, stage, N, h, j, acc);
    } else {
      for (int k0 = 0; k0 < K; k0 += kc) {
        const int cur = min(kc, K - k0);
        __syncthreads();
        stage_weights(W, N, k0, cur, stage);
        __syncthreads();
        if (rb < nrb) gemm_accumulate_chunk<NB>(Xrow + k0, row_ok, cur, stage, N, h, j, acc);
      }
    }
    if (rb < nrb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int orow = p0 + rb * 32 + 8 * (r / 4) + 4 * h + (r % 4);
        if (orow < p1) {
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
            const float v = acc[nb][r];
            if (slab) slab[(orow - p0) * N + nb * 32 + j] = v;
            if (T && orow >= wb0 && orow < wb1) T[(size_t)orow * N + nb * 32 + j] = v;
          }
        }
      }
    }
  }
}

// Fused GeMM-SpMM tile kernel: phase 1 is the tile GEMM into the LDS slab, phase 2 the
// consumer rows out of LDS (same as the SpMM-SpMM kernel).
template <int NB, int LPR>
__global__ __launch_bounds__(kBlock) void fused_gemm_spmm_kernel(
    const TileDesc *__restrict__ tiles, int n_tiles, int per_xcd, const int *__restrict__ fused_ids,
    const float *__restrict__ B, const float *__restrict__ C, int K, int kc, const int *__restrict__ Ap,
    const int *__restrict__ Ai, const float *__restrict__ Ax, float *__restrict__ D,
    float *__restrict__ T, int accumulate) {
  extern __shared__ __align__(16) float lds[];
  constexpr int N = NB * 32;
  constexpr int V = 4;
  const int tile = xcd_contiguous(blockIdx.x, per_xcd);
  if (tile >= n_tiles) return;
  const TileDesc t = tiles[tile];
  float *stage = lds;
  float *slab = lds + kc * N;
  const bool has_cons = t.cons_end > t.cons_begin;
  tile_gemm<NB>(B, C, K, kc, t.prod_begin, t.prod_end, stage, has_cons ? slab : nullptr,
                t.wb_end > t.wb_begin ? T : nullptr, t.wb_begin, t.wb_end);
  if (!has_cons) return;
  __syncthreads();
  constexpr int G = kBlock / LPR;
  const int group = threadIdx.x / LPR, glane = threadIdx.x % LPR;
  const int coff = glane * V;
  const bool ok = coff < N;
  const LdsRows<V> tsrc{slab, N, ok ? coff : 0, t.prod_begin};
  for (int q = t.cons_begin + group; q < t.cons_end; q += G) {
    const int i = fused_ids[q];
    fvec<V> acc = vzero<V>();
    if (accumulate && ok) acc = *reinterpret_cast<const fvec<V> *>(D + (size_t)i * N + coff);
    row_dot<V, LPR>(Ai, Ax, Ap[i], Ap[i + 1], glane, ok, tsrc, acc);
    if (ok) store_streaming<V>(D + (size_t)i * N + coff, acc);
  }
}

// Plain GEMM  Y = X * W  (tf_gemm) when K*N is too large to keep W in LDS: 128 rows per
// workgroup, W streamed through LDS in kc-row slices.
template <int NB>
__global__ __launch_bounds__(kBlock) void gemm_kernel(const float *__restrict__ X, const float *__restrict__ W,
                                                      float *__restrict__ Y, int M, int K, int kc,
                                                      int per_xcd, int n_blocks) {
  extern __shared__ __align__(16) float lds[];
  const int b = xcd_contiguous(blockIdx.x, per_xcd);
  if (b >= n_blocks) return;
  const int p0 = b * 128, p1 = min(M, p0 + 128);
  tile_gemm<NB>(X, W, K, kc, p0, p1, lds, nullptr, Y, p0, p1);
}

// Row-list GEMM  Y[r,:] = X[r,:K] * W  for r = rows[q] (or r = q when rows is null):
// intermediate rows that no tile fuses, and tf_gemm.  Persistent: W (K x N) is copied to
// LDS once per workgroup, then every wavefront walks its own 32-row blocks with no
// barrier at all; the rows of X for the next 32 values of k are already in flight
// (16 bytes per lane and load, see tile_gemm for the k permutation) while the MFMAs of
// the current ones issue.
constexpr int kGemmBlock = 512;

template <int NB> struct alignas((NB == 1 || NB == 2 || NB == 4) ? 4 * NB : (NB == 8 ? 16 : 4)) wvec { float v[NB]; };

// Column block nb of a wavefront's 32 x (32 NB) output tile holds the columns NB j + nb, j = 0 .. 31 (not
// 32 nb + j): W then sits in LDS as it is in memory, row-major, the NB values a lane feeds to the NB MFMAs of
// one k step are adjacent (one LDS read of 4 NB bytes per k step), and a lane ends up with NB consecutive
// columns of each of its output rows, which leave with one store (16 bytes when NB = 4; a row of the tile
// is 32 such stores side by side).  The reads for the next eight values of k are issued before the MFMAs
// of the current eight.
template <int NB>
__device__ __forceinline__ void mfma_step8(const fvec<4> &a, const wvec<NB> (&bw)[4], v16f (&acc)[NB]) {
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
      acc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[t], bw[t].v[nb], acc[nb], 0, 0, 0);
}

// Copies W (K x N, row-major) into LDS as it is: 16 bytes per load, eight loads in flight per thread.
template <int NB>
__device__ __forceinline__ void stage_weights(const float *__restrict__ W, int K, float *wlds) {
  constexpr int N = NB * 32;
  const int n4 = K * N / 4;
  const fvec<4> *src = reinterpret_cast<const fvec<4> *>(W);
  fvec<4> *dst = reinterpret_cast<fvec<4> *>(wlds);
  for (int i0 = threadIdx.x; i0 < n4; i0 += 8 * kGemmBlock) {
    fvec<4> v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kGemmBlock;
      v[u] = src[i < n4 ? i : i0];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kGemmBlock;
      if (i < n4) dst[i] = v[u];
    }
  }
}

constexpr int kGemmSeg = 16;  // row blocks whose row numbers a wavefront keeps in LDS at a time

// G4C > 0: K = 32 G4C is known when the kernel is built, and a block's MFMAs, the requests for the operands
// three groups ahead and the reads of W one step ahead are one stretch of code without a branch: a wavefront
// issues in order, so address arithmetic, a wait for a row number or a branch between two MFMAs leaves the
// pipe without work from this wavefront (39,000 -> 33,500 cycles per block and wavefront for K = 128, of
// which the block's 256 MFMAs of the two wavefronts of a SIMD take 32,800).
// YPOS (row lists only): the result of list position q goes to row q of Y instead of row rows[q] -- the rows of the
// result stored side by side in the order of the list.
template <int NB, bool LIST, int G4C, bool YPOS = false>
__global__ __launch_bounds__(kGemmBlock) void gemm_rows_kernel(const float *__restrict__ X,
                                                               const float *__restrict__ W,
                                                               float *__restrict__ Y,
                                                               const int *__restrict__ rows, int n_rows,
                                                               int K) {
  extern __shared__ __align__(16) float wlds[];
  constexpr int N = NB * 32;
  stage_weights<NB>(W, K, wlds);
  __syncthreads();
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int h = lane / 32, j = lane % 32;
  const int total_waves = gridDim.x * (kGemmBlock / 64);
  const int nrb = (n_rows + 31) / 32;
  const int steps = K / 8;  // 8-wide k steps; this lane's rows of W in step s are 8s + 4h + t
  const int G4 = (steps + 3) / 4;  // groups of four steps (32 values of k): the unit the A operand is fetched in
  const wvec<NB> *wl = reinterpret_cast<const wvec<NB> *>(wlds) + (4 * h) * 32 + j;
  // this wavefront's slice of LDS behind W: the row numbers of the blocks it is working on (row
  // lists only).  Reading them from LDS keeps the row list out of the chain of global loads, so
  // the A operands requested ahead are never waited for early.
  int *ridx = reinterpret_cast<int *>(wlds + K * N) + wave * (kGemmSeg * 32);
  // every wavefront walks one contiguous run of row blocks; run lengths differ by at most one
  // and the longer runs are spread evenly over the compute units
  const int gw = blockIdx.x * (kGemmBlock / 64) + wave;
  // When the blocks do not divide among the wavefronts, the odd ones are cut into their NB column blocks
  // and those are dealt out instead: a wavefront with one more whole block than the others would set
  // the kernel's time (200,000 rows are 6,250 blocks for 2,048 wavefronts: four blocks against three
  // and a quarter).  Not when the odd blocks are so many that a wavefront would get all columns anyway.
  const int whole = nrb / total_waves, odd = nrb - whole * total_waves;
  const int tail_per_wave = (odd * NB + total_waves - 1) / total_waves;
  const bool split_tail = odd > 0 && tail_per_wave < NB;
  const int run0 = split_tail ? gw * whole : (int)((long long)gw * nrb / total_waves);
  const int run_end = split_tail ? run0 + whole : (int)((long long)(gw + 1) * nrb / total_waves);
  if (split_tail) {
    const int n_tail = odd * NB;
    for (int t = gw * tail_per_wave; t < min(n_tail, (gw + 1) * tail_per_wave); ++t) {
      const int rb = whole * total_waves + t / NB, nb = t % NB;
      const int pos = min(rb * 32 + j, n_rows - 1);
      const float *p = X + (size_t)(LIST ? rows[pos] : pos) * K + 4 * h;
      v16f acc1;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc1[r] = 0.f;
      const float *wt = wlds + ((4 * h) * 32 + j) * NB + nb;  // W[k][NB j + nb] sits at (k*32 + j)*NB + nb
      fvec<4> a = *reinterpret_cast<const fvec<4> *>(p);
      for (int st = 0; st < steps; ++st) {
        const fvec<4> an = *reinterpret_cast<const fvec<4> *>(p + 8 * min(st + 1, steps - 1));
#pragma unroll
        for (int u = 0; u < 4; ++u)
          acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[u], wt[(size_t)(8 * st + u) * 32 * NB], acc1, 0, 0, 0);
        a = an;
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int x = rb * 32 + 8 * (r / 4) + 4 * h + (r % 4);
        if (x < n_rows) Y[(size_t)(LIST && !YPOS ? rows[x] : x) * N + NB * j + nb] = acc1[r];
      }
    }
  }
  for (int rb0 = run0; rb0 < run_end; rb0 += kGemmSeg) {
    const int rb_end = min(run_end, rb0 + kGemmSeg);
    if constexpr (LIST) {
      for (int x = lane; x < (rb_end - rb0) * 32; x += 64) ridx[x] = rows[min(rb0 * 32 + x, n_rows - 1)];
    }
    const int total_groups = (rb_end - rb0) * G4;
    // row (of X and Y) behind position x of this segment
    auto row_at = [&](int x) { return LIST ? ridx[x] : min(rb0 * 32 + x, n_rows - 1); };
    // ... and the row of Y it is stored to
    auto yrow_at = [&](int x) { return LIST && !YPOS ? ridx[x] : min(rb0 * 32 + x, n_rows - 1); };
    if constexpr (G4C > 0) {
      static_assert(G4C >= 4 && G4C % 4 == 0, "four operand sets in turn, a block starts with the first");
      const int nblk = rb_end - rb0;
      auto operand_row = [&](int b) { return X + (size_t)row_at(min(b, nblk - 1) * 32 + j) * K + 4 * h; };
      const float *pc = operand_row(0);
      fvec<4> set[4][4];
#pragma unroll
      for (int q = 0; q < 3; ++q)
#pragma unroll
        for (int u = 0; u < 4; ++u) set[q][u] = load4(pc + q * 32 + 8 * u);
      wvec<NB> bw[4], bn[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) bw[t] = wl[t * 32];
      // accumulator register r of block b, all NB column blocks, into its row of Y
      auto store_row = [&](const v16f (&acc)[NB], int b, int r) __attribute__((always_inline)) {
        wvec<NB> out;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) out.v[nb] = acc[nb][r];
        *reinterpret_cast<wvec<NB> *>(Y + (size_t)yrow_at(b * 32 + 8 * (r / 4) + 4 * h + (r % 4)) * N + NB * j) = out;
      };
      for (int b = 0; b < nblk; ++b) {
        const float *pn = operand_row(b + 1);
        v16f acc[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[nb][r] = 0.f;
#pragma unroll
        for (int g = 0; g < G4C; ++g) {
          const float *src = g + 3 < G4C ? pc + (g + 3) * 32 : pn + (g + 3 - G4C) * 32;
#pragma unroll
          for (int u = 0; u < 4; ++u) set[(g + 3) % 4][u] = load4(src + 8 * u);
          __builtin_amdgcn_sched_barrier(0);  // the requests stay here: the scheduler would move them to the block's end
#pragma unroll
          for (int t2 = 0; t2 < 4; t2 += 2) {
            const int st = 4 * g + t2;
#pragma unroll
            for (int t = 0; t < 4; ++t) bn[t] = wl[(8 * (st + 1) + t) * 32];
            mfma_step8<NB>(set[g % 4][t2], bw, acc);
#pragma unroll
            for (int t = 0; t < 4; ++t) bw[t] = wl[(8 * ((st + 2) % (4 * G4C)) + t) * 32];
            mfma_step8<NB>(set[g % 4][t2 + 1], bn, acc);
          }
        }
        if ((rb0 + b + 1) * 32 <= n_rows) {
#pragma unroll
          for (int r = 0; r < 16; ++r) store_row(acc, b, r);
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if ((rb0 + b) * 32 + 8 * (r / 4) + 4 * h + (r % 4) < n_rows) store_row(acc, b, r);
        }
        pc = pn;
      }
      continue;
    }
    // A operand of group gi (block rb0 + gi / G4, steps 4 (gi % G4) ..): four 16-byte loads per lane,
    // always issued (block and k clamped to existing ones, the surplus is never used) so that the
    // loads of later groups stay in flight while earlier ones are consumed.
    auto load_group = [&](int gi, fvec<4> (&c)[4]) {
      const int g = min(gi, total_groups - 1);
      const int s0 = (g % G4) * 4;
      const float *p = X + (size_t)row_at((g / G4) * 32 + j) * K + s0 * 8 + 4 * h;
#pragma unroll
      for (int u = 0; u < 4; ++u) c[u] = *reinterpret_cast<const fvec<4> *>(p + 8 * min(u, steps - 1 - s0));
    };
    // three register sets, used in turn: a group's operands are requested two groups ahead
    fvec<4> set0[4], set1[4], set2[4];
    load_group(0, set0);
    load_group(1, set1);
    v16f acc[NB];
    auto run_group = [&](int gi, const fvec<4> (&c)[4]) {
      const int g = gi % G4, blk = gi / G4, s0 = 4 * g;
      if (g == 0) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[nb][r] = 0.f;
      }
      wvec<NB> bw[4], bn[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) bw[t] = wl[(8 * s0 + t) * 32];
      {
        const int sn = min(s0 + 1, steps - 1);
#pragma unroll
        for (int t = 0; t < 4; ++t) bn[t] = wl[(8 * sn + t) * 32];
        mfma_step8<NB>(c[0], bw, acc);
      }
      if (s0 + 1 < steps) {
        const int sn = min(s0 + 2, steps - 1);
#pragma unroll
        for (int t = 0; t < 4; ++t) bw[t] = wl[(8 * sn + t) * 32];
        mfma_step8<NB>(c[1], bn, acc);
      }
      if (s0 + 2 < steps) {
        const int sn = min(s0 + 3, steps - 1);
#pragma unroll
        for (int t = 0; t < 4; ++t) bn[t] = wl[(8 * sn + t) * 32];
        mfma_step8<NB>(c[2], bw, acc);
      }
      if (s0 + 3 < steps) mfma_step8<NB>(c[3], bn, acc);
      if (g == G4 - 1) {
        // accumulator register r of column block nb of lane (h, j) holds output row 8*(r/4) + 4*h + r%4, column NB j + nb
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int x = blk * 32 + 8 * (r / 4) + 4 * h + (r % 4);
          if (rb0 * 32 + x < n_rows) {
            wvec<NB> out;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) out.v[nb] = acc[nb][r];
            *reinterpret_cast<wvec<NB> *>(Y + (size_t)yrow_at(x) * N + NB * j) = out;
          }
        }
      }
    };
    for (int gi = 0; gi < total_groups; gi += 3) {
      load_group(gi + 2, set2);
      run_group(gi, set0);
      if (gi + 1 < total_groups) {
        load_group(gi + 3, set0);
        run_group(gi + 1, set1);
      }
      if (gi + 2 < total_groups) {
        load_group(gi + 4, set1);
        run_group(gi + 2, set2);
      }
    }
  }
}

// Fused GeMM-SpMM tile kernel with W in registers.  v_mfma_f32_16x16x4_f32: a wavefront
// owns 16 output columns (CPW such column blocks when N > 128) and keeps its K x 16 slice of
// W in registers for the whole tile -- lane (j = lane%16, h = lane/16) holds
// W[16m + 4h + u][16*cb + j] in w[4m + u] -- so LDS holds the slab of intermediate rows and
// a small staging buffer for X, and two workgroups share a compute unit: one runs its MFMA
// phase while the other gathers its fused rows out of LDS.
// X reaches the MFMAs through LDS: the workgroup copies 64 rows x 32 values of k at a time
// (one 16-byte load per thread, whole cache lines per row) into one of two buffers, two
// chunks ahead in registers; every wavefront then reads its A operands from there, 16 bytes
// per lane and four MFMA steps per read: lane (j, h) reads X[row0 + j][16m + 4h .. +4), and
// both operands use the same permuted k order.  The slab's row stride is N + 4 floats and
// the staging buffer's 36, which keeps the lanes of a read or store in different banks.
typedef float v4f __attribute__((ext_vector_type(4)));
constexpr int kSlabPad = 4;
constexpr int kXRows = 64, kXChunk = 32, kXLd = kXChunk + 4;
constexpr int kXStageFloats = 2 * kXRows * kXLd;  // both buffers

template <int KS, int CPW, int LPR>
__global__ __launch_bounds__(kGemmBlock) void fused_gemm_spmm_regw_kernel(
    const TileDesc *__restrict__ tiles, int n_tiles, int per_xcd, const int *__restrict__ fused_ids,
    const float *__restrict__ B, const float *__restrict__ W, int K, int N, const int *__restrict__ Ap,
    const int *__restrict__ Ai, const float *__restrict__ Ax, float *__restrict__ D, float *__restrict__ T,
    int accumulate) {
  extern __shared__ __align__(16) float lds[];
  static_assert(kGemmBlock * 4 == kXRows * kXChunk, "one 16-byte unit of a chunk per thread");
  const int tile = xcd_contiguous(blockIdx.x, per_xcd);
  if (tile >= n_tiles) return;
  const TileDesc t = tiles[tile];
  constexpr int NW = kGemmBlock / 64;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int j = lane % 16, h = lane / 16;
  const int CB = N / 16;  // column blocks
  // N <= 64 (LPR <= 16): RG wavefronts share a column block and split the four row blocks of a chunk
  constexpr int RG = CPW == 1 ? (LPR == 8 ? 4 : LPR == 16 ? 2 : 1) : 1;
  const int cb0 = RG > 1 ? wave % (NW / RG) : wave;
  const int rg = RG > 1 ? wave / (NW / RG) : 0;
  const int ld = N + kSlabPad;
  const int P = t.prod_end - t.prod_begin;
  const int R = t.cons_end - t.cons_begin;
  const bool has_cons = R > 0;
  constexpr int V = 4;
  constexpr int G = kGemmBlock / LPR;
  constexpr int RND = 8;  // fused rows per lane group whose entries are fetched ahead of the MFMA phase
  const int group = threadIdx.x / LPR, glane = threadIdx.x % LPR;
  float *xbuf = lds;
  float *slab = lds + kXStageFloats;
  // (row, first entry, end) of every fused row of the tile, behind the slab
  int4 *cinfo = reinterpret_cast<int4 *>(slab + P * ld);
  for (int x = threadIdx.x; x < R; x += kGemmBlock) {
    const int i = fused_ids[t.cons_begin + x];
    cinfo[x] = make_int4(i, Ap[i], Ap[i + 1], 0);
  }

  // staging role of this thread: 16 bytes of row sr of every chunk
  const int sr = threadIdx.x / 8, sk = (threadIdx.x % 8) * 4;
  const int nkc = (K + kXChunk - 1) / kXChunk;
  const int nchunks = ((P + kXRows - 1) / kXRows) * nkc;
  auto chunk_unit = [&](int ch) -> fvec<4> {
    const int q = ch / nkc, k = (ch % nkc) * kXChunk + sk;
    const int row = t.prod_begin + min(q * kXRows + sr, P - 1);  // rows past the end repeat the last one
    return (ch < nchunks && k < K) ? *reinterpret_cast<const fvec<4> *>(B + (size_t)row * K + k) : vzero<4>();
  };
  fvec<4> x0 = chunk_unit(0), x1 = chunk_unit(1), x2 = chunk_unit(2);

  float w[CPW][KS * 4];
  if (cb0 < CB) {  // uniform per wavefront
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      const int cb = cb0 + NW * c;
#pragma unroll
      for (int m = 0; m < KS; ++m)
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int k = 16 * m + 4 * h + u;
          w[c][4 * m + u] = (cb < CB && k < K) ? W[(size_t)k * N + 16 * cb + j] : 0.f;
        }
    }
  }
  *reinterpret_cast<fvec<4> *>(xbuf + sr * kXLd + sk) = x0;
  x0 = x1;
  x1 = x2;
  __syncthreads();  // chunk 0 and cinfo visible
  // The first LPR entries of the rows this lane group will compute are requested now and used
  // after the MFMA phase: their latency is covered by it.
  int pc[RND];
  float pa[RND];
#pragma unroll
  for (int r = 0; r < RND; ++r) {
    pc[r] = 0;
    pa[r] = 0.f;
    const int x = r * G + group;
    if (x < R) {
      const int4 ci = cinfo[x];
      const int k = ci.y + glane;
      if (k < ci.z) { pc[r] = Ai[k]; pa[r] = Ax[k]; }
    }
  }

  int ch = 0;
  for (int r0 = 0; r0 < P; r0 += kXRows) {
    v4f acc[CPW][4];
#pragma unroll
    for (int c = 0; c < CPW; ++c)
#pragma unroll
      for (int b = 0; b < 4; ++b) acc[c][b] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kc = 0; kc < KS / 2; ++kc) {
      if (kc * kXChunk < K) {  // uniform
        x2 = chunk_unit(ch + 3);
        const float *xb = xbuf + (ch & 1) * (kXRows * kXLd);
        if (cb0 < CB) {
#pragma unroll
          for (int m2 = 0; m2 < 2; ++m2) {
            fvec<4> a[4];
#pragma unroll
            for (int bi = 0; bi < 4; ++bi)
              if (bi * RG < 4)
                a[bi] = *reinterpret_cast<const fvec<4> *>(xb + (16 * (rg + RG * bi) + j) * kXLd + 16 * m2 + 4 * h);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
              for (int bi = 0; bi < 4; ++bi)
                if (bi * RG < 4) {
#pragma unroll
                  for (int c = 0; c < CPW; ++c)
                    acc[c][bi] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[bi].v[u], w[c][4 * (2 * kc + m2) + u],
                                                                      acc[c][bi], 0, 0, 0);
                }
          }
        }
        if (ch + 1 < nchunks)
          *reinterpret_cast<fvec<4> *>(xbuf + ((ch + 1) & 1) * (kXRows * kXLd) + sr * kXLd + sk) = x0;
        x0 = x1;
        x1 = x2;
        ++ch;
        __syncthreads();
      }
    }
    // accumulator register r of lane (j, h) is output row 4h + r, column j of its block
    if (cb0 < CB) {
#pragma unroll
      for (int bi = 0; bi < 4; ++bi)
        if (bi * RG < 4) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int lr = r0 + 16 * (rg + RG * bi) + 4 * h + r;
            if (lr < P) {
              const int row = t.prod_begin + lr;
              const bool wb = row >= t.wb_begin && row < t.wb_end;
#pragma unroll
              for (int c = 0; c < CPW; ++c) {
                const int col = 16 * (cb0 + NW * c) + j;
                if (col < N) {
                  if (has_cons) slab[lr * ld + col] = acc[c][bi][r];
                  if (wb) T[(size_t)row * N + col] = acc[c][bi][r];
                }
              }
            }
          }
        }
    }
  }
  if (!has_cons) return;
  __syncthreads();
  const int coff = glane * V;
  const bool ok = coff < N;
  const LdsRows<V> tsrc{slab, ld, ok ? coff : 0, t.prod_begin};
#pragma unroll
  for (int r = 0; r < RND; ++r) {
    const int x = r * G + group;
    if (x < R) {  // uniform per lane group
      const int4 ci = cinfo[x];
      fvec<V> acc = vzero<V>();
      if (accumulate && ok) acc = *reinterpret_cast<const fvec<V> *>(D + (size_t)ci.x * N + coff);
      row_dot_loaded<V, LPR>(pc[r], pa[r], min(LPR, ci.z - ci.y), ok, tsrc, acc);
      row_dot<V, LPR>(Ai, Ax, ci.y + LPR, ci.z, glane, ok, tsrc, acc);
      if (ok) store_streaming<V>(D + (size_t)ci.x * N + coff, acc);
    }
  }
  for (int x = RND * G + group; x < R; x += G) {
    const int4 ci = cinfo[x];
    fvec<V> acc = vzero<V>();
    if (accumulate && ok) acc = *reinterpret_cast<const fvec<V> *>(D + (size_t)ci.x * N + coff);
    row_dot<V, LPR>(Ai, Ax, ci.y, ci.z, glane, ok, tsrc, acc);
    if (ok) store_streaming<V>(D + (size_t)ci.x * N + coff, acc);
  }
}

// Streaming fused GeMM-SpMM kernel.  A workgroup walks one long run of intermediate rows,
// 64 at a time, and keeps only the last `ring_rows` of them in LDS (a ring: row r sits in
// slot (r - prod_begin) % ring_rows).  Eight producer wavefronts compute the next 64 rows on
// MFMA exactly as in the tile kernel above (W in registers, X through the staging buffers)
// while NCW consumer wavefronts compute the fused rows whose last column was produced in
// the step before -- the schedule lists them step by step -- so the MFMA pipe and the
// VALU/LDS gather work overlap all the time, W is loaded once per run and no row is computed
// twice inside a run.  Both kinds of wavefront meet at one barrier per 32 values of k
// (the staging rhythm: KS/2 intervals per step, the ones past K empty); the consumers spread
// a step's rows evenly over those intervals.
// Nothing that is still in flight is ever moved between registers: a producer thread keeps
// one staging register per interval of a step (a whole step of X in flight), the barriers
// wait for LDS traffic only, and a consumer lane group
// keeps one register set per interval of a step -- the (row, first entry, end) record of the
// row it will compute in the same interval of the next step is requested a step ahead, its
// first LPR entries half a step ahead, both unconditionally (clamped to existing records).  The entries are turned
// into (byte offset into the ring, value) pairs in a small per-group LDS area and walked in
// CSR order with broadcast reads.
constexpr int kStreamProducers = 8;   // wavefronts

template <int KS, int CPW, int LPR, int NCW, bool ACC>
__global__ __launch_bounds__((kStreamProducers + NCW) * 64) void fused_gemm_spmm_stream_kernel(
    const TileDesc *__restrict__ tiles, const int *__restrict__ step_begin, const int *__restrict__ step_ptr,
    const int4 *__restrict__ fused_rec, const float *__restrict__ B, const float *__restrict__ W, int K, int N,
    int ring_rows, const int *__restrict__ Ai, const float *__restrict__ Ax, float *__restrict__ D,
    float *__restrict__ T, int relu_in) {
  extern __shared__ __align__(16) float lds[];
  const TileDesc t = tiles[blockIdx.x];
  constexpr int NW = kStreamProducers;
  constexpr int NKC = KS / 2;  // intervals per step
  static_assert(NKC % 2 == 0, "the two LDS staging buffers alternate by interval parity");
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int ld = N + kSlabPad;
  const int P = t.prod_end - t.prod_begin;
  const int S = (P + kXRows - 1) / kXRows;  // production steps
  float *xbuf = lds;
  float *ring = lds + kXStageFloats;
  const int ring_mask = ring_rows - 1;
  int *sp = reinterpret_cast<int *>(ring + ring_rows * ld) + NCW * 128;  // S + 2 offsets into fused_rec
  for (int x = threadIdx.x; x < S + 2; x += (NW + NCW) * 64) sp[x] = step_ptr[step_begin[blockIdx.x] + x];

  if (wave < NW) {
    // ---- producers -------------------------------------------------------------------
    const int j = lane % 16, h = lane / 16;
    const int CB = N / 16;
    constexpr int RG = CPW == 1 ? (LPR == 8 ? 4 : LPR == 16 ? 2 : 1) : 1;
    const int cb0 = RG > 1 ? wave % (NW / RG) : wave;
    const int rg = RG > 1 ? wave / (NW / RG) : 0;
    const int sr = threadIdx.x / 8, sk = (threadIdx.x % 8) * 4;
    // Always a load (of the last row / the last values of k when past the end, zeroed when it
    // is stored to LDS): a load under a condition would have to land before the next barrier.
    auto chunk_unit = [&](int ch) -> fvec<4> {
      const int q = min(ch / NKC, S - 1), k = min((ch % NKC) * kXChunk + sk, K - 4);
      const int row = t.prod_begin + min(q * kXRows + sr, P - 1);
      return load_streaming4(B + (size_t)row * K + k);
    };
    // relu_in: B is a layer's output before its activation, max(x, 0) is applied here on its way to the MFMAs
    // (the second layer of tf_gcn_two_layers: saves a pass over the hidden layer)
    auto unit_or_zero = [&](const fvec<4> &x, int kc) -> fvec<4> {
      fvec<4> r = kc * kXChunk + sk < K ? x : vzero<4>();
      if (relu_in) {
#pragma unroll
        for (int c = 0; c < 4; ++c) r.v[c] = fmaxf(r.v[c], 0.f);
      }
      return r;
    };
    float *const xdst = xbuf + sr * kXLd + sk;
    const int ld4 = ld * 4;
    char *const ring_lane = reinterpret_cast<char *>(ring) + ((16 * rg + 4 * h) * ld + 16 * cb0 + j) * 4;
    {
      const fvec<4> first = chunk_unit(0);
      *reinterpret_cast<fvec<4> *>(xdst) = unit_or_zero(first, 0);
    }
    fvec<4> xs[NKC];  // xs[k]: the unit of the next interval k of a step that is not in LDS yet
#pragma unroll
    for (int k = 0; k < NKC; ++k) xs[(k + 1) % NKC] = chunk_unit(k + 1);
    float w[CPW][KS * 4];
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
      const int cb = cb0 + NW * c;
#pragma unroll
      for (int m = 0; m < KS; ++m)
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int k = 16 * m + 4 * h + u;
          w[c][4 * m + u] = (cb < CB && k < K) ? W[(size_t)k * N + 16 * cb + j] : 0.f;
        }
    }
    // W has landed before the loop starts.  (Otherwise the first MFMA of every step waits for "everything
    // requested before this point" -- the compiler cannot tell the loads of W, long done, from the staging
    // unit requested a moment ago, and a step would begin by waiting out a full trip to memory.)
#pragma unroll
    for (int c = 0; c < CPW; ++c)
#pragma unroll
      for (int i = 0; i < KS * 4; ++i) asm volatile("" : : "v"(w[c][i]));
    lds_barrier();
    for (int q = 0; q < S; ++q) {
      v4f acc[CPW][4];
#pragma unroll
      for (int c = 0; c < CPW; ++c)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[c][b] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kc = 0; kc < NKC; ++kc) {
        const int ch = q * NKC + kc;
        const float *xb = xbuf + (kc & 1) * (kXRows * kXLd);
        if (cb0 < CB && kc * kXChunk < K) {  // uniform
#pragma unroll
          for (int m2 = 0; m2 < 2; ++m2) {
            fvec<4> a[4];
#pragma unroll
            for (int bi = 0; bi < 4; ++bi)
              if (bi * RG < 4)
                a[bi] = *reinterpret_cast<const fvec<4> *>(xb + (16 * (rg + RG * bi) + j) * kXLd + 16 * m2 + 4 * h);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
              for (int bi = 0; bi < 4; ++bi)
                if (bi * RG < 4) {
#pragma unroll
                  for (int c = 0; c < CPW; ++c)
                    acc[c][bi] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[bi].v[u], w[c][4 * (2 * kc + m2) + u],
                                                                      acc[c][bi], 0, 0, 0);
                }
          }
        }
        // the unit of the next interval goes to the other buffer, its register takes the unit
        // of the same interval of the next step
        *reinterpret_cast<fvec<4> *>(xdst + ((kc + 1) & 1) * (kXRows * kXLd)) = unit_or_zero(xs[(kc + 1) % NKC], (kc + 1) % NKC);
        xs[(kc + 1) % NKC] = chunk_unit(ch + 1 + NKC);
        if (kc == NKC - 1 && cb0 < CB) {
          // last interval of the step: the 64 new rows go into the ring (and to HBM where the
          // remainder reads them) before the barrier that lets the consumers at them
          const int row0 = t.prod_begin + q * kXRows;
          const bool plain = (q + 1) * kXRows <= P && (row0 + kXRows <= t.wb_begin || row0 >= t.wb_end);
          if (plain) {
            // a whole step without a row to write back (all but a run's ends): sixteen stores off one address.
            // A step's 64 rows never wrap in the ring (its size is a multiple of 64), so only the step's first
            // slot is reduced; everything else is this lane's fixed place in the step plus a multiple of a row.
            char *base = ring_lane + ((q * kXRows) & ring_mask) * ld4;
#pragma unroll
            for (int bi = 0; bi < 4; ++bi)
              if (bi * RG < 4) {
#pragma unroll
                for (int r = 0; r < 4; ++r)
#pragma unroll
                  for (int c = 0; c < CPW; ++c)
                    *reinterpret_cast<float *>(base + (16 * RG * bi + r) * ld4 + 64 * NW * c) = acc[c][bi][r];
              }
          } else {
#pragma unroll
            for (int bi = 0; bi < 4; ++bi)
              if (bi * RG < 4) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                  const int lr = q * kXRows + 16 * (rg + RG * bi) + 4 * h + r;
                  if (lr < P) {
                    const int row = t.prod_begin + lr;
                    const bool wb = row >= t.wb_begin && row < t.wb_end;
#pragma unroll
                    for (int c = 0; c < CPW; ++c) {
                      const int col = 16 * (cb0 + NW * c) + j;
                      if (col < N) {
                        ring[(lr & ring_mask) * ld + col] = acc[c][bi][r];
                        if (wb) T[(size_t)row * N + col] = acc[c][bi][r];
                      }
                    }
                  }
                }
              }
          }
        }
        lds_barrier();
      }
    }
    return;
  }

  // ---- consumers -----------------------------------------------------------------------
  constexpr int NG = NCW * 64 / LPR;  // lane groups = fused rows in flight
  const int ctid = threadIdx.x - NW * 64;
  const int cg = ctid / LPR, glane = ctid % LPR;
  const int coff = glane * 4;
  const bool ok = coff < N;
  int2 *scratch = reinterpret_cast<int2 *>(ring + ring_rows * ld) + cg * LPR;
  const char *rbase = reinterpret_cast<const char *>(ring) + (ok ? coff : 0) * 4;
  lds_barrier();  // step table visible (the producers' first staging unit too)
  const int sp_first = sp[0], sp_last = sp[S + 1];
  // Rows of a step [c0, c0 + len) handled in its interval kc: an even share.
  auto share = [&](int c0, int len, int kc, int &b, int &e) {
    b = c0 + len * kc / NKC;
    e = c0 + len * (kc + 1) / NKC;
  };
  // The record is loaded whether or not the interval has a row for this lane group (the index
  // is clamped into the run's records): a load under a condition would have to land before
  // the next barrier, an unconditional one stays in flight.  The row is used only if it exists.
  const int rec_first = sp_first, rec_last = sp_last - 1;
  auto load_rec = [&](int c0, int len, int kc, int r) -> int4 {
    int b, e;
    share(c0, len, kc, b, e);
    return fused_rec[min(max(b + cg + NG * r, rec_first), rec_last)];
  };
  // A fused row of a streamed schedule has at most EPL * LPR entries (32, or 64 when N > 128
  // -- the inspector sees to it) and a step has at most NG rows per interval: the steady
  // state below has no loop and no conditional load, so the loads it issues ahead of time
  // are waited for only when their registers are read.
  constexpr int EPL = LPR >= 32 ? 1 : 32 / LPR;  // entries of a row per lane
  auto row = [&](const int4 rec, const int (&c)[EPL], const float (&a)[EPL]) {
    fvec<4> acc = vzero<4>();
    float *dst = D + (size_t)rec.x * N + coff;
    if constexpr (ACC) { if (ok) acc = *reinterpret_cast<const fvec<4> *>(dst); }
#pragma unroll
    for (int u = 0; u < EPL; ++u) {
      const int cnt = min(LPR, rec.z - rec.y - u * LPR);
      if (u == 0 || cnt > 0) {
        scratch[glane] = make_int2(((c[u] - t.prod_begin) & ring_mask) * (ld * 4), __float_as_int(a[u]));
        acc = lds_row_dot_quad(scratch, 0, cnt, rbase, glane & 3, acc);  // (reads up to 3 pairs past the row's: never used)
      }
    }
    if (ok) store_streaming<4>(dst, acc);
  };
  // Entries glane, glane + LPR, .. of a row (lanes past the row's end re-read its last entry;
  // the row's length decides what is used).
  auto load_entries = [&](const int4 r, int (&c)[EPL], float (&a)[EPL]) {
#pragma unroll
    for (int u = 0; u < EPL; ++u) {
      const int k = min(r.y + u * LPR + glane, r.z - 1);
      c[u] = Ai[k];
      a[u] = Ax[k];
    }
  };
  constexpr int AHEAD = NKC / 2;  // a record is requested NKC intervals ahead, its entries AHEAD
  // rows a lane group computes per interval so that a step's 64 new rows are taken in one step
  constexpr int RPI = (kXRows + NG * NKC - 1) / (NG * NKC);
  int4 rec[NKC][RPI];
  int pc[NKC][RPI][EPL];
  float pa[NKC][RPI][EPL];
#pragma unroll
  for (int kc = 0; kc < NKC; ++kc)
#pragma unroll
    for (int r = 0; r < RPI; ++r) rec[kc][r] = load_rec(sp_first, sp[1] - sp_first, kc, r);
#pragma unroll
  for (int kc = 0; kc < AHEAD; ++kc)
#pragma unroll
    for (int r = 0; r < RPI; ++r) load_entries(rec[kc][r], pc[kc][r], pa[kc][r]);
  int s0 = sp_first, s1 = sp[1];  // rows of step q are [s0, s1)
  for (int q = 0; q < S; ++q) {
    const int s2 = q + 1 < S ? sp[q + 2] : s1;  // rows of the next production step: [s1, s2)
#pragma unroll
    for (int kc = 0; kc < NKC; ++kc) {
      int4 cur[RPI];
      int c[RPI][EPL];
      float a[RPI][EPL];
#pragma unroll
      for (int r = 0; r < RPI; ++r) {
        cur[r] = rec[kc][r];
#pragma unroll
        for (int u = 0; u < EPL; ++u) { c[r][u] = pc[kc][r][u]; a[r][u] = pa[kc][r][u]; }
      }
      constexpr int NKC_ = NKC;
      const int kp = (kc + AHEAD) % NKC_;
#pragma unroll
      for (int r = 0; r < RPI; ++r) {
        load_entries(rec[kp][r], pc[kp][r], pa[kp][r]);
        rec[kc][r] = load_rec(s1, s2 - s1, kc, r);
      }
      int b, e;
      share(s0, s1 - s0, kc, b, e);
#pragma unroll
      for (int r = 0; r < RPI; ++r)
        if (b + cg + NG * r < e) row(cur[r], c[r], a[r]);
      lds_barrier();
    }
    s0 = s1;
    s1 = s2;
  }
  // rows whose last column came with the last step
  for (int x = sp[S] + cg; x < sp[S + 1]; x += NG) {
    const int4 r = fused_rec[x];
    int c[EPL];
    float a[EPL];
    load_entries(r, c, a);
    row(r, c, a);
  }
}

// ---------------------------------------------------------------------------------
// Fused SpMM-SpMM over marching runs (stencils on 3D grids): one workgroup of 32 lane groups
// walks a run iteration by iteration.  LDS holds numbered slots of one 64-column row each; the
// schedule has turned every column index into the byte offset of the slot that holds the row
// at that time, so the kernel knows nothing of grids or stencils:
//   iteration i   rows of C of load list i are in their slots
//                 ELL rows [row_ptr[2i], row_ptr[2i+1]): intermediate rows, summed from slots of C
//                 into the slot ~out; barrier;
//                 ELL rows [row_ptr[2i+1], row_ptr[2i+2]): rows `out` of D, summed from slots of
//                 the intermediate; the rows of C of list i+1, held in registers meanwhile, go to
//                 their slots (whose last readers have run); barrier.
// An ELL row is 8 (offset, value) pairs, 64 bytes: the lanes of a quad hold two pairs each and
// pass them on by DPP; padding pairs read a row of zeros with value 0.  Entries are walked in
// CSR order, so results carry the reference's bits.
// Memory latency is what such a loop has to hide: a run is one workgroup per compute unit, in
// step with all others.  The lists of an iteration (its ELL rows and the load list two lists
// on) are requested two iterations ahead and the rows of C two lists ahead, into register
// sets used in turn -- which is why the workgroup has 512 threads: eight wavefronts have 256
// registers each.  Loads return in the order they were issued, so within an iteration what is
// needed first is requested first.
// ---------------------------------------------------------------------------------
constexpr int kMarchBlock = kMarchGroups * 16;

// -1 / 0 for true / false, in a form the compiler cannot see through: a value that was loaded and is
// blended with such a mask stays a load that is always issued.  (Written as a select, the load moves
// under the condition, and a load under a condition is waited for at once.)
__device__ __forceinline__ int opaque_mask(bool c) {
  int m = c ? -1 : 0;
  asm volatile("" : "+v"(m));
  return m;
}

// The lists are read once: streaming loads, so that they do not push the rows of C out of L2.
__device__ __forceinline__ int4 load_streaming_i4(const int4 *p) {
  typedef int i4 __attribute__((ext_vector_type(4)));
  const i4 v = __builtin_nontemporal_load(reinterpret_cast<const i4 *>(p));
  return make_int4(v[0], v[1], v[2], v[3]);
}

// Loads at a uniform base plus a 32-bit byte offset per lane: the address is formed by the load itself (scalar
// base + vector offset) instead of by 64-bit arithmetic on the VALU, which a wavefront of this kernel pays for in
// cycles it would otherwise issue FMAs in.  (The schedule is only built for operands these offsets reach.)
__device__ __forceinline__ int4 march_load_i4_nt(const void *base, unsigned off) {
  return load_streaming_i4(reinterpret_cast<const int4 *>(reinterpret_cast<const char *>(base) + off));
}
__device__ __forceinline__ int march_load_i(const void *base, unsigned off) {
  return *reinterpret_cast<const int *>(reinterpret_cast<const char *>(base) + off);
}
__device__ __forceinline__ int2 march_load_i2(const void *base, unsigned off) {
  return *reinterpret_cast<const int2 *>(reinterpret_cast<const char *>(base) + off);
}
__device__ __forceinline__ fvec<4> march_load_f4(const void *base, unsigned off) {
  return load4(reinterpret_cast<const float *>(reinterpret_cast<const char *>(base) + off));
}
// row * row_bytes + lane_off for row < 2^24, row_bytes < 2^24 and a product below 2^32: one full-rate instruction
__device__ __forceinline__ unsigned march_row_off(int row, unsigned row_bytes, unsigned lane_off) {
  return __umul24((unsigned)row, row_bytes) + lane_off;
}

template <int G>
__device__ __forceinline__ fvec<4> march_gather(const char *lane_base, int off) {
  return *reinterpret_cast<const fvec<4> *>(lane_base + quad_bcast<G>(off));
}

// One ELL row: the lanes of a quad hold two (LDS offset, value) pairs each.  Four gathers are in
// flight at a time (eight measured no faster and cost sixteen registers).
// W: the longest row of either pattern, 5 .. 8: a 7-point stencil's rows never fill the eighth pair, a
// 5-point stencil's not the last three, which then are neither gathered nor multiplied.
template <int W>
__device__ __forceinline__ fvec<4> march_row(const int4 e, const char *lane_base) {
  static_assert(W >= 5 && W <= 8, "pairs 0 .. 4 are always taken");
  fvec<4> x[4];
  x[0] = march_gather<0>(lane_base, e.x); x[1] = march_gather<0>(lane_base, e.z);
  x[2] = march_gather<1>(lane_base, e.x); x[3] = march_gather<1>(lane_base, e.z);
  fvec<4> acc = vzero<4>();
  quad_fma<0>(e.y, x[0], acc); quad_fma<0>(e.w, x[1], acc);
  x[0] = march_gather<2>(lane_base, e.x);
  if constexpr (W > 5) x[1] = march_gather<2>(lane_base, e.z);
  quad_fma<1>(e.y, x[2], acc); quad_fma<1>(e.w, x[3], acc);
  if constexpr (W > 6) x[2] = march_gather<3>(lane_base, e.x);
  if constexpr (W > 7) x[3] = march_gather<3>(lane_base, e.z);
  quad_fma<2>(e.y, x[0], acc);
  if constexpr (W > 5) quad_fma<2>(e.w, x[1], acc);
  if constexpr (W > 6) quad_fma<3>(e.y, x[2], acc);
  if constexpr (W > 7) quad_fma<3>(e.w, x[3], acc);
  return acc;
}

// The same for rows of up to 32 entries: a lane of the 16-lane group holds two (LDS offset, value) pairs, lane l the
// pairs 2l and 2l + 1, and a pair reaches the group's other lanes through a DPP row broadcast (row_newbcast: the value
// of one lane of every row of sixteen).  Entry j's gather address is one v_add_u32 with the broadcast as its operand,
// its four FMAs take the broadcast value as theirs.  Four gathers in flight; entries in CSR order.
template <int L> __device__ __forceinline__ unsigned march_bcast_add(int off, unsigned lane_addr) {
  unsigned r;
  asm("s_nop 1\n\t"
      "v_add_u32_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf"
      : "=v"(r)
      : "v"(off), "v"(lane_addr), "n"(L));
  return r;
}
template <int L> __device__ __forceinline__ void march_bcast_fma(int val, const fvec<4> &x, fvec<4> &acc) {
  asm("s_nop 1\n\t"
      "v_fmac_f32_dpp %0, %4, %5 row_newbcast:%9 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %1, %4, %6 row_newbcast:%9 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %2, %4, %7 row_newbcast:%9 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %3, %4, %8 row_newbcast:%9 row_mask:0xf bank_mask:0xf"
      : "+v"(acc.v[0]), "+v"(acc.v[1]), "+v"(acc.v[2]), "+v"(acc.v[3])
      : "v"(val), "v"(x.v[0]), "v"(x.v[1]), "v"(x.v[2]), "v"(x.v[3]), "n"(L));
}
__device__ __forceinline__ fvec<4> march_lds_read(unsigned addr) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  const f4 v = *reinterpret_cast<const __attribute__((address_space(3))) f4 *>(addr);
  fvec<4> r;
  r.v[0] = v[0]; r.v[1] = v[1]; r.v[2] = v[2]; r.v[3] = v[3];
  return r;
}
template <int J, int W>
__device__ __forceinline__ void march_wide_gather4(const int4 e, unsigned lane_addr, fvec<4> (&x)[4]) {
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    if (J + u < W) {
      // (J is a multiple of 4: entries J, J+1 sit in lane J/2, entries J+2, J+3 in lane J/2 + 1)
      if (u == 0) x[0] = march_lds_read(march_bcast_add<J / 2>(e.x, lane_addr));
      if (u == 1) x[1] = march_lds_read(march_bcast_add<J / 2>(e.z, lane_addr));
      if (u == 2) x[2] = march_lds_read(march_bcast_add<J / 2 + 1>(e.x, lane_addr));
      if (u == 3) x[3] = march_lds_read(march_bcast_add<J / 2 + 1>(e.z, lane_addr));
    }
  }
}
template <int J, int W>
__device__ __forceinline__ void march_wide_fma4(const int4 e, const fvec<4> (&x)[4], fvec<4> &acc) {
  if (J + 0 < W) march_bcast_fma<J / 2>(e.y, x[0], acc);
  if (J + 1 < W) march_bcast_fma<J / 2>(e.w, x[1], acc);
  if (J + 2 < W) march_bcast_fma<J / 2 + 1>(e.y, x[2], acc);
  if (J + 3 < W) march_bcast_fma<J / 2 + 1>(e.w, x[3], acc);
}
template <int B, int NB, int W>
__device__ __forceinline__ void march_wide_blocks(const int4 e, unsigned lane_addr, fvec<4> (&cur)[4], fvec<4> (&nxt)[4], fvec<4> &acc) {
  if constexpr (B < NB) {
    if constexpr (B + 1 < NB) march_wide_gather4<4 * (B + 1), W>(e, lane_addr, nxt);
    march_wide_fma4<4 * B, W>(e, cur, acc);
    march_wide_blocks<B + 1, NB, W>(e, lane_addr, nxt, cur, acc);
  }
}
template <int W>
__device__ __forceinline__ fvec<4> march_row_wide(const int4 e, unsigned lane_addr) {
  static_assert(W >= 9 && W <= 32, "rows of up to 8 entries take the quad layout");
  fvec<4> xa[4], xb[4];
  fvec<4> acc = vzero<4>();
  march_wide_gather4<0, W>(e, lane_addr, xa);
  march_wide_blocks<0, (W + 3) / 4, W>(e, lane_addr, xa, xb, acc);
  return acc;
}

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// What a lane keeps of one iteration's lists: its pairs of the ELL rows of its lane group (up to
// kMarchTpg intermediate rows, kMarchDpg second-op rows), where they go, and the group's share
// of the load list two lists on.
struct MarchLists {
  int4 et[kMarchTpg], ed[kMarchDpg];
  int ot[kMarchTpg], od[kMarchDpg];
  int2 ll[kMarchLpg];
};
// Rows of C on their way: the group's share of one load list and the rows themselves.
struct MarchStage {
  int2 ll[kMarchLpg];
  fvec<4> c[kMarchLpg];
};

template <bool ACC, int W, bool WIDE = false>
__global__ __launch_bounds__(kMarchBlock) void fused_spmm_spmm_march_kernel(
    const int2 *__restrict__ runs, int n_runs, int per_xcd, const int *__restrict__ row_ptr,
    const int *__restrict__ load_ptr, const int2 *__restrict__ load_list, const int *__restrict__ row_out,
    const int4 *__restrict__ ell, const float *__restrict__ C, float *__restrict__ D, float *__restrict__ trash, int N) {
  extern __shared__ __align__(16) unsigned char smem[];
  char *lds = reinterpret_cast<char *>(smem);
  const int run = xcd_contiguous(blockIdx.x, per_xcd);
  if (run >= n_runs) return;
  const int2 rd = runs[run];
  const int n_iter = rd.y;
  // per iteration i = 0..n_iter: [4i] first intermediate row, [4i+1] first second-op row, [4i+2] first load
  int *tab = reinterpret_cast<int *>(lds);
  for (int i = threadIdx.x; i <= n_iter; i += kMarchBlock) {
    const int g = rd.x + i;
    tab[4 * i] = row_ptr[2 * g];
    tab[4 * i + 1] = i < n_iter ? row_ptr[2 * g + 1] : 0;
    tab[4 * i + 2] = load_ptr[g];
  }
  if (threadIdx.x < 16) *reinterpret_cast<fvec<4> *>(lds + kMarchZeroOff + threadIdx.x * 16) = vzero<4>();
  __syncthreads();
  const int group = threadIdx.x >> 4, glane = threadIdx.x & 15, q = threadIdx.x & 3;
  // an ELL row is 64 bytes, four lanes of a quad take 16 each -- or 256 bytes, sixteen lanes of the group take 16 each
  const unsigned q16 = (WIDE ? glane : q) * 16, row_bytes = (unsigned)N * 4;
  constexpr int ELLS = WIDE ? 8 : 6;  // log2 of an ELL row's bytes
  char *lane_base = lds + glane * 16;
  const unsigned lane_addr = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char *)lane_base;
  auto ell_row = [&](const int4 e) __attribute__((always_inline)) {
    if constexpr (WIDE) return march_row_wide<W>(e, lane_addr);
    else return march_row<W>(e, lane_base);
  };
  // List entries [b, e) dealt to the lane groups.  Nothing in the loop is under a condition: a lane
  // group without an entry loads row 0 of C into the trash row, computes a row of padding into the
  // trash row, stores it to the trash row in global memory.  A wait for an older load can then leave
  // all younger ones in flight, which loads and stores under conditions do not allow.
  auto fetch_loads = [&](int list, int2 (&l)[kMarchLpg]) {
    const bool in = list < n_iter;
    const int b = in ? tab[4 * list + 2] : 0, e = in ? tab[4 * list + 6] : 0;
#pragma unroll
    for (int u = 0; u < kMarchLpg; ++u) {
      const int x = b + group + kMarchGroups * u;
      const int2 v = march_load_i2(load_list, (unsigned)max(min(x, e - 1), 0) << 3);
      const int m = opaque_mask(x < e);
      l[u] = make_int2(v.x, (v.y & m) | (kMarchTrashOff & ~m));  // a group without an entry re-reads another's row into the trash row
    }
  };
  auto fetch_lists = [&](int it, MarchLists &L) {
    const bool in = it < n_iter;
    const int b0 = in ? tab[4 * it] : 0, b1 = in ? tab[4 * it + 1] : 0, b2 = in ? tab[4 * it + 4] : 0;
#pragma unroll
    for (int u = 0; u < kMarchTpg; ++u) {
      const int x = b0 + group + kMarchGroups * u, xc = max(min(x, b1 - 1), 0);
      const bool ok = x < b1;
      const int o = march_load_i(row_out, (unsigned)xc << 2), m = opaque_mask(ok);
      L.et[u] = march_load_i4_nt(ell, ((unsigned)xc << ELLS) + q16);  // a group without a row recomputes another's, into the trash row
      L.ot[u] = (o & m) | (~kMarchTrashOff & ~m);
    }
#pragma unroll
    for (int u = 0; u < kMarchDpg; ++u) {
      const int x = b1 + group + kMarchGroups * u, xc = max(min(x, b2 - 1), 0);
      const bool ok = x < b2;
      const int o = march_load_i(row_out, (unsigned)xc << 2), m = opaque_mask(ok);
      L.ed[u] = march_load_i4_nt(ell, ((unsigned)xc << ELLS) + q16);
      L.od[u] = o | ~m;  // -1: no row
    }
    fetch_loads(it + 2, L.ll);
  };

  for (int c0 = 0; c0 < N; c0 += 64) {
    const unsigned lane_off = (c0 + glane * 4) * 4;  // this lane's four columns of the strip, in bytes
    float *Dl = D + c0 + glane * 4;
    float *Tl = trash + glane * 4;
    // (plain loads: a run's rows of C are its neighbours' halo rows an iteration or two later, and
    // after a streaming load they were gone from L2 by then -- 1.36 GB fetched per launch on the 128^3
    // grid against 1.05 GB)
    auto issue = [&](MarchStage &S) {
#pragma unroll
      for (int u = 0; u < kMarchLpg; ++u) S.c[u] = march_load_f4(C, march_row_off(S.ll[u].x, row_bytes, lane_off));
    };
    // One iteration.  `cur` holds its lists; `fut` is free and takes those of iteration it + 2.  Stage
    // X is free (its rows went to LDS an iteration ago) and takes list it + 2, whose entries came with
    // `cur`; stage Y holds list it + 1, which goes to LDS in the second half.  The requests to memory
    // are dealt out over the rows, one share before each row: all at once at the top of the iteration
    // they queue at the memory pipeline while the LDS and the ALUs have nothing to do.
    auto step = [&](int it, const MarchLists &cur, MarchLists &fut, MarchStage &X, const MarchStage &Y) __attribute__((always_inline)) {
      static_assert(kMarchLpg == kMarchTpg + kMarchDpg, "one share of the requests per row");
      const int nx = it + 2, nl = it + 4;
      const bool in = nx < n_iter, inl = nl < n_iter;
      const int b0 = in ? tab[4 * nx] : 0, b1 = in ? tab[4 * nx + 1] : 0, b2 = in ? tab[4 * nx + 4] : 0;
      const int lb = inl ? tab[4 * nl + 2] : 0, le = inl ? tab[4 * nl + 6] : 0;
      auto share = [&](auto vc) __attribute__((always_inline)) {
        constexpr int v = decltype(vc)::value;
        X.ll[v] = cur.ll[v];
        X.c[v] = march_load_f4(C, march_row_off(X.ll[v].x, row_bytes, lane_off));
        if constexpr (v < kMarchTpg) {
          const int x = b0 + group + kMarchGroups * v, xc = max(min(x, b1 - 1), 0);
          const int o = march_load_i(row_out, (unsigned)xc << 2), m = opaque_mask(x < b1);
          fut.et[v] = march_load_i4_nt(ell, ((unsigned)xc << ELLS) + q16);  // a group without a row recomputes another's, into the trash row
          fut.ot[v] = (o & m) | (~kMarchTrashOff & ~m);
        } else {
          constexpr int u = v - kMarchTpg;
          const int x = b1 + group + kMarchGroups * u, xc = max(min(x, b2 - 1), 0);
          const int o = march_load_i(row_out, (unsigned)xc << 2), m = opaque_mask(x < b2);
          fut.ed[u] = march_load_i4_nt(ell, ((unsigned)xc << ELLS) + q16);
          fut.od[u] = o | ~m;  // -1: no row
        }
        const int x = lb + group + kMarchGroups * v;
        const int2 l = march_load_i2(load_list, (unsigned)max(min(x, le - 1), 0) << 3);
        const int m = opaque_mask(x < le);
        fut.ll[v] = make_int2(l.x, (l.y & m) | (kMarchTrashOff & ~m));  // a group without an entry re-reads another's row into the trash row
      };
      // the intermediate rows this iteration's second-op rows are the first to read
      static_for<0, kMarchTpg>([&](auto uc) {
        constexpr int u = decltype(uc)::value;
        share(uc);
        const fvec<4> acc = ell_row(cur.et[u]);
        *reinterpret_cast<fvec<4> *>(lane_base + ~cur.ot[u]) = acc;
      });
      lds_barrier();
      // the second-op rows; the next rows of C take the slots of rows no one reads any more
      static_for<0, kMarchDpg>([&](auto uc) {
        constexpr int u = decltype(uc)::value;
        share(std::integral_constant<int, kMarchTpg + u>{});
        fvec<4> acc = ell_row(cur.ed[u]);
        float *dst = cur.od[u] >= 0 ? Dl + (size_t)cur.od[u] * N : Tl;
        if (ACC) vadd<4>(*reinterpret_cast<const fvec<4> *>(dst), acc);
        store_streaming<4>(dst, acc);
      });
#pragma unroll
      for (int u = 0; u < kMarchLpg; ++u) *reinterpret_cast<fvec<4> *>(lane_base + Y.ll[u].y) = Y.c[u];
      lds_barrier();
    };
    MarchLists E0, E1, E2;
    MarchStage S0, S1;
    // before the first iteration: its rows of C into their slots (a list of any length), list 1 on its
    // way, the lists of the first two iterations
    fetch_lists(0, E0);
    fetch_loads(1, S1.ll);
    fetch_lists(1, E1);
    for (int x = tab[2] + group; x < tab[6]; x += kMarchGroups) {
      const int2 l = load_list[x];
      *reinterpret_cast<fvec<4> *>(lane_base + l.y) = march_load_f4(C, march_row_off(l.x, row_bytes, lane_off));
    }
    issue(S1);
    __syncthreads();
    // (six steps, the period of the register sets, without a way out in between: iterations past the
    // run's last find empty lists and work on the trash rows.  A path that skips steps would make
    // the waits for loads assume that nothing younger is in flight.)
    for (int it = 0; it < n_iter; it += 6) {
      step(it, E0, E2, S0, S1);
      step(it + 1, E1, E0, S1, S0);
      step(it + 2, E2, E1, S0, S1);
      step(it + 3, E0, E2, S1, S0);
      step(it + 4, E1, E0, S0, S1);
      step(it + 5, E2, E1, S1, S0);
    }
  }
}

// ell[e] = (LDS offset, value): the value of entry src[e] of B, or of A when kMarchSrcA is set; 0 for padding.
__global__ void march_fill_kernel(const int *__restrict__ off, const int *__restrict__ src, const float *__restrict__ Ax,
                                  const float *__restrict__ Bx, int2 *__restrict__ ell, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const int sidx = src[i];
    float v = 0.f;
    if (sidx >= 0) v = (sidx & kMarchSrcA) ? Ax[sidx & (kMarchSrcA - 1)] : Bx[sidx];
    ell[i] = make_int2(off[i], __float_as_int(v));
  }
}

// ---------------------------------------------------------------------------------
// Host-side launchers
// ---------------------------------------------------------------------------------
namespace {

struct Shape { int V, LPR; };

Shape pick_shape(int N) {
  int V = (N % 4 == 0) ? 4 : (N % 2 == 0) ? 2 : 1;
  int lanes = (N + V - 1) / V;
  int LPR = 8;
  while (LPR < lanes && LPR < 64) LPR *= 2;
  return {V, LPR};
}

// Work items per XCD for xcd_contiguous; 0 (identity mapping) when the environment variable
// TF_XCD_REMAP is set to 0.  The grid is sized grid_of(n) either way.
inline bool xcd_remap_on() {
  static const bool on = [] { const char *e = getenv("TF_XCD_REMAP"); return !(e && e[0] == '0'); }();
  return on;
}
inline int per_xcd_of(int n) { return xcd_remap_on() ? (n + kXcds - 1) / kXcds : 0; }
inline int grid_of(int n) { return (n + kXcds - 1) / kXcds * kXcds; }
// The same for chunks of `bpc` items per XCD turn (see xcd_contiguous).
inline int chunk_bpc(int n, int bpc) { return !xcd_remap_on() ? 0 : (bpc <= 0 || bpc * kXcds >= n) ? (n + kXcds - 1) / kXcds : bpc; }
inline int grid_chunked(int n, int bpc) { return bpc <= 0 ? grid_of(n) : (n + bpc * kXcds - 1) / (bpc * kXcds) * (bpc * kXcds); }

template <class F> hipError_t allow_lds(F kernel, int bytes) {
  if (bytes <= 65536) return hipSuccess;
  return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                             hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

#define TF_DISPATCH_VL(V_, L_, CALL)                                         \
  do {                                                                       \
    if (V_ == 4) {                                                           \
      if (L_ == 8) { CALL(4, 8); } else if (L_ == 16) { CALL(4, 16); }       \
      else if (L_ == 32) { CALL(4, 32); } else { CALL(4, 64); }              \
    } else if (V_ == 2) {                                                    \
      if (L_ == 8) { CALL(2, 8); } else if (L_ == 16) { CALL(2, 16); }       \
      else if (L_ == 32) { CALL(2, 32); } else { CALL(2, 64); }              \
    } else {                                                                 \
      if (L_ == 8) { CALL(1, 8); } else if (L_ == 16) { CALL(1, 16); }       \
      else if (L_ == 32) { CALL(1, 32); } else { CALL(1, 64); }              \
    }                                                                        \
  } while (0)

#define TF_DISPATCH_NB(NB_, CALL)                                            \
  do {                                                                       \
    switch (NB_) {                                                           \
      case 1: CALL(1); break; case 2: CALL(2); break; case 3: CALL(3); break; \
      case 4: CALL(4); break; case 5: CALL(5); break; case 6: CALL(6); break; \
      case 7: CALL(7); break; default: CALL(8); break;                       \
    }                                                                        \
  } while (0)

}  // namespace

hipError_t launch_fused_spmm_spmm(const TileDesc *tiles, int n_tiles, const int *fused_ids,
                                  const int *Bp, const int *Bi, const float *Bx, const float *C,
                                  const int *Ap, const int *Ai, const float *Ax, float *D, float *T,
                                  int N, int lds_bytes, int accumulate, hipStream_t st) {
  if (n_tiles <= 0) return hipSuccess;
  const Shape s = pick_shape(N);
  const int per = per_xcd_of(n_tiles);
  hipError_t err = hipSuccess;
#define CALL(V_, L_)                                                                       \
  err = allow_lds(fused_spmm_spmm_kernel<V_, L_>, lds_bytes);                              \
  if (err == hipSuccess)                                                                   \
    hipLaunchKernelGGL((fused_spmm_spmm_kernel<V_, L_>), dim3(grid_of(n_tiles)), dim3(kBlock),   \
                       lds_bytes, st, tiles, n_tiles, per, fused_ids, Bp, Bi, Bx, C, Ap, Ai, \
                       Ax, D, T, N, N, accumulate)
  TF_DISPATCH_VL(s.V, s.LPR, CALL);
#undef CALL
  return err != hipSuccess ? err : hipGetLastError();
}

#ifndef TF_WIN_BLOCK
#define TF_WIN_BLOCK 512
#endif
hipError_t launch_fused_spmm_spmm_window(const TileDesc *tiles, const int *win, int n_tiles,
                                         const int *fused_ids, const int *Bp, const int *Bi,
                                         const float *Bx, const float *C, float *D, int N, int strip,
                                         int lds_bytes, int accumulate, hipStream_t st) {
  if (n_tiles <= 0) return hipSuccess;
  constexpr int BLOCK = TF_WIN_BLOCK;
  const int per = per_xcd_of(n_tiles);
  const int2 *w2 = reinterpret_cast<const int2 *>(win);
  hipError_t err;
#define CALLW(SW_, ACC_)                                                                               \
  err = allow_lds(fused_spmm_spmm_window_kernel<SW_, BLOCK, ACC_>, lds_bytes);                         \
  if (err == hipSuccess)                                                                               \
    hipLaunchKernelGGL((fused_spmm_spmm_window_kernel<SW_, BLOCK, ACC_>), dim3(grid_of(n_tiles)), dim3(BLOCK), \
                       lds_bytes, st, tiles, w2, n_tiles, per, fused_ids, Bp, Bi, Bx, C, D, N)
  if (strip == 32) {
    if (accumulate) { CALLW(32, true); } else { CALLW(32, false); }
  } else {
    if (accumulate) { CALLW(64, true); } else { CALLW(64, false); }
  }
#undef CALLW
  return err != hipSuccess ? err : hipGetLastError();
}

hipError_t launch_fused_spmm_spmm_window64(const TileDesc *tiles, const int *win, int n_tiles, const int *Bp,
                                           const int *Bi, const float *Bx, int nnzB, const float *C, const int *Ap,
                                           const int *Ai, const float *Ax, int nnzA, float *D, int N, int lds_bytes,
                                           int accumulate, int compute_units, hipStream_t st) {
  if (n_tiles <= 0) return hipSuccess;
  // wavefronts that fetch the next strip's window during the second product: two are enough for one
  // more strip of one tile per compute unit, four keep up when tiles or strips queue
  const int n_loaders = (n_tiles > compute_units || N > 2 * kW64Strip) ? 4 : 2;
  if (N % kW64Strip != 0 || nnzA < 4 || nnzB < 4 || nnzA >= (1 << 30) || nnzB >= (1 << 30)) return hipErrorInvalidValue;
  const int per = per_xcd_of(n_tiles);
  const int2 *w2 = reinterpret_cast<const int2 *>(win);
  hipError_t err;
#define CALL64(ACC_)                                                                                    \
  err = allow_lds(fused_spmm_spmm_window64_kernel<ACC_>, lds_bytes);                                    \
  if (err == hipSuccess)                                                                                \
    hipLaunchKernelGGL((fused_spmm_spmm_window64_kernel<ACC_>), dim3(grid_of(n_tiles)), dim3(kW64Block), \
                       lds_bytes, st, tiles, w2, n_tiles, per, Bp, Bi, Bx, nnzB, C, Ap, Ai, Ax, nnzA, D, N, n_loaders)
  if (accumulate) { CALL64(true); } else { CALL64(false); }
#undef CALL64
  return err != hipSuccess ? err : hipGetLastError();
}

hipError_t launch_spmm_rows(const int *rows, int n_rows, const int *Ap, const int *Ai, const float *Ax,
                            const float *X, float *Y, int N, int accumulate, int xcd_chunk_rows,
                            int streaming, hipStream_t st, int compact, int coalesced_pairs, int flagged) {
  if (n_rows <= 0) return hipSuccess;
  const Shape s = pick_shape(N);
  if (flagged && s.V != 4) return hipErrorInvalidValue;  // (schedules mark columns only when N is a multiple of 4)
  const int G = kBlock / s.LPR;
  const int n_blocks = (n_rows + G - 1) / G;
  // 0: workgroup b takes block b; > 0: chunks of rows per XCD turn; < 0: one contiguous run per XCD
  const int bpc = xcd_chunk_rows == 0 ? 0 : chunk_bpc(n_blocks, xcd_chunk_rows > 0 ? std::max(1, xcd_chunk_rows / G) : 0);
#define CALL3(V_, L_, COAL_, FLAG_)                                                                                   \
  hipLaunchKernelGGL((spmm_rows_kernel<V_, L_, COAL_, FLAG_>), dim3(grid_chunked(n_blocks, bpc)), dim3(kBlock), 0, st, \
                     rows, n_rows, n_blocks, bpc, Ap, Ai, Ax, X, N, Y, N, accumulate, streaming, compact)
#define CALL2(V_, L_, COAL_) CALL3(V_, L_, COAL_, false)
#define CALL(V_, L_) do { if (coalesced_pairs) { CALL2(V_, L_, true); } else { CALL2(V_, L_, false); } } while (0)
#define CALLF(L_) do { if (coalesced_pairs) { CALL3(4, L_, true, true); } else { CALL3(4, L_, false, true); } } while (0)
  if (flagged) {
    if (s.LPR == 8) { CALLF(8); } else if (s.LPR == 16) { CALLF(16); } else if (s.LPR == 32) { CALLF(32); } else { CALLF(64); }
    return hipGetLastError();
  }
  TF_DISPATCH_VL(s.V, s.LPR, CALL);
#undef CALL
#undef CALL2
#undef CALL3
#undef CALLF
  return hipGetLastError();
}

hipError_t launch_long_rows(const LongChunk *chunks, int n_chunks, const LongRow *rows, int n_long,
                            const int *Ai, const float *Ax, const float *X, float *partial, float *Y,
                            int N, int accumulate, hipStream_t st) {
  if (n_chunks <= 0) return hipSuccess;
  const Shape s = pick_shape(N);
#define CALL(V_, L_)                                                                          \
  hipLaunchKernelGGL((spmm_long_chunk_kernel<V_, L_>), dim3(n_chunks), dim3(kBlock), 0, st,   \
                     chunks, Ai, Ax, X, N, partial, N)
  TF_DISPATCH_VL(s.V, s.LPR, CALL);
#undef CALL
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(long_row_reduce_kernel, dim3(n_long), dim3(kBlock), 0, st, rows, partial, Y, N,
                     accumulate);
  return hipGetLastError();
}

// Long rows regrouped by column partition.  The executor runs the hot segments (an eighth per
// XCD, in XCD order) on the row kernel with one contiguous run of segments per XCD and the cold
// ones round-robin; these two put A's values into segment order and add up a row's segments.
hipError_t launch_scatter_values(const int *ent_src, const int *ent_pos, const float *Ax, float *seg_val, int n_entries,
                                 hipStream_t st) {
  if (n_entries <= 0) return hipSuccess;
  const int blocks = std::min((n_entries + kBlock - 1) / kBlock, 65536);
  hipLaunchKernelGGL(scatter_values_kernel, dim3(blocks), dim3(kBlock), 0, st, ent_src, ent_pos, Ax, seg_val, n_entries);
  return hipGetLastError();
}

hipError_t launch_gather_values(const int *src, const float *Ax, float *out, int n, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  const int blocks = std::min((n + kBlock - 1) / kBlock, 65536);
  hipLaunchKernelGGL(gather_values_kernel, dim3(blocks), dim3(kBlock), 0, st, src, Ax, out, n);
  return hipGetLastError();
}

// Y[rows[q].row] (+)= the sums in partial[seg_of[first .. first + count)], in that order (Y may be
// `partial` itself for the groups of segments of rows with many).
hipError_t launch_seg_reduce(const LongRow *rows, int n_rows, const int *seg_of, const float *partial, float *Y, int N,
                             int accumulate, hipStream_t st) {
  if (n_rows <= 0) return hipSuccess;
  const Shape s = pick_shape(N);
  const int G = kBlock / s.LPR;
#define CALL(V_, L_)                                                                                                \
  hipLaunchKernelGGL((long_seg_reduce_kernel<V_, L_>), dim3((n_rows + G - 1) / G), dim3(kBlock), 0, st, rows, n_rows, \
                     seg_of, partial, Y, N, accumulate)
  TF_DISPATCH_VL(s.V, s.LPR, CALL);
#undef CALL
  return hipGetLastError();
}

hipError_t launch_fused_gemm_spmm(const TileDesc *tiles, int n_tiles, const int *fused_ids,
                                  const float *B, const float *C, int K, int kc, const int *Ap,
                                  const int *Ai, const float *Ax, float *D, float *T, int N,
                                  int lds_bytes, int accumulate, int compute_units, int regw,
                                  hipStream_t st) {
  if (n_tiles <= 0) return hipSuccess;
  const int per = per_xcd_of(n_tiles);
  const int NB = N / 32;
  const int LPR = pick_shape(N).LPR;
  hipError_t err = hipSuccess;
  if (regw) {
    // W in registers: K <= 16*KS values of k per lane, CPW column blocks of 16 per wavefront
    const int KS = K <= 64 ? 4 : K <= 128 ? 8 : 16;
    const int CPW = N > 128 ? 2 : 1;
    if (K > 256 || N > 256 || KS * CPW > 16) return hipErrorInvalidValue;
#define CALL3(KS_, CPW_, L_)                                                                       \
  err = allow_lds(fused_gemm_spmm_regw_kernel<KS_, CPW_, L_>, lds_bytes);                          \
  if (err == hipSuccess)                                                                           \
    hipLaunchKernelGGL((fused_gemm_spmm_regw_kernel<KS_, CPW_, L_>), dim3(grid_of(n_tiles)),       \
                       dim3(kGemmBlock), lds_bytes, st, tiles, n_tiles, per, fused_ids, B, C, K, N, \
                       Ap, Ai, Ax, D, T, accumulate)
#define CALL2(KS_)                                                             \
  do {                                                                         \
    if (CPW == 2) { if constexpr (KS_ <= 8) { CALL3(KS_, 2, 64); } }           \
    else if (LPR == 8) { CALL3(KS_, 1, 8); }                                   \
    else if (LPR == 16) { CALL3(KS_, 1, 16); }                                 \
    else { CALL3(KS_, 1, 32); }                                                \
  } while (0)
    if (KS == 4) CALL2(4); else if (KS == 8) CALL2(8); else CALL2(16);
#undef CALL2
#undef CALL3
    return err != hipSuccess ? err : hipGetLastError();
  }
#define CALL2(NB_, L_)                                                                      \
  err = allow_lds(fused_gemm_spmm_kernel<NB_, L_>, lds_bytes);                              \
  if (err == hipSuccess)                                                                    \
    hipLaunchKernelGGL((fused_gemm_spmm_kernel<NB_, L_>), dim3(grid_of(n_tiles)), dim3(kBlock),   \
                       lds_bytes, st, tiles, n_tiles, per, fused_ids, B, C, K, kc, Ap, Ai, Ax, \
                       D, T, accumulate)
#define CALL(NB_)                                                         \
  do {                                                                    \
    if (LPR == 8) { CALL2(NB_, 8); } else if (LPR == 16) { CALL2(NB_, 16); } \
    else if (LPR == 32) { CALL2(NB_, 32); } else { CALL2(NB_, 64); }      \
  } while (0)
  TF_DISPATCH_NB(NB, CALL);
#undef CALL
#undef CALL2
  return err != hipSuccess ? err : hipGetLastError();
}

hipError_t launch_fused_gemm_spmm_stream(const TileDesc *tiles, int n_tiles, const int *step_begin,
                                         const int *step_ptr, const int *fused_rec, const float *B,
                                         const float *C, int K, int N, int ring_rows, const int *Ai,
                                         const float *Ax, float *D, float *T, int lds_bytes, int accumulate,
                                         hipStream_t st, int relu_in) {
  if (n_tiles <= 0) return hipSuccess;
  const int LPR = pick_shape(N).LPR;
  const int KS = K <= 64 ? 4 : K <= 128 ? 8 : 16;
  const int CPW = N > 128 ? 2 : 1;
  if (K > 256 || N > 128 || CPW != 1 || ring_rows < 256 || (ring_rows & (ring_rows - 1))) return hipErrorInvalidValue;
  hipError_t err = hipSuccess;
  const int4 *rec = reinterpret_cast<const int4 *>(fused_rec);
  // eight consumer wavefronts when the producers' registers allow sixteen wavefronts, else four
#define CALL4(KS_, L_, NCW_, ACC_)                                                                   \
  err = allow_lds(fused_gemm_spmm_stream_kernel<KS_, 1, L_, NCW_, ACC_>, lds_bytes);                 \
  if (err == hipSuccess)                                                                             \
    hipLaunchKernelGGL((fused_gemm_spmm_stream_kernel<KS_, 1, L_, NCW_, ACC_>), dim3(n_tiles),       \
                       dim3((kStreamProducers + NCW_) * 64), lds_bytes, st, tiles, step_begin, step_ptr, \
                       rec, B, C, K, N, ring_rows, Ai, Ax, D, T, relu_in)
#define CALL3(KS_, L_, NCW_)                                                   \
  do { if (accumulate) { CALL4(KS_, L_, NCW_, true); } else { CALL4(KS_, L_, NCW_, false); } } while (0)
#define CALL2(KS_, NCW_)                                                       \
  do {                                                                         \
    if (LPR == 8) { CALL3(KS_, 8, NCW_); }                                     \
    else if (LPR == 16) { CALL3(KS_, 16, NCW_); }                              \
    else { CALL3(KS_, 32, NCW_); }                                             \
  } while (0)
  if (KS == 4) CALL2(4, 8); else if (KS == 8) CALL2(8, 8); else CALL2(16, 4);
#undef CALL2
#undef CALL3
#undef CALL4
  return err != hipSuccess ? err : hipGetLastError();
}

hipError_t launch_gemm(const float *X, const float *W, float *Y, const int *rows, int n_rows, int K,
                       int N, int compute_units, hipStream_t st, int y_by_position) {
  if (n_rows <= 0) return hipSuccess;
  if (y_by_position && !rows) return hipErrorInvalidValue;
  const int NB = N / 32;
  hipError_t err = hipSuccess;
  const int w_bytes = K * N * 4;
  if (w_bytes <= 131072) {
    // W resident in LDS: persistent workgroups, as many per compute unit as the LDS allows
    const int per_cu = 1;  // register use (accumulators + both operand pipelines) allows one 8-wave workgroup
    const int nrb = (n_rows + 31) / 32;
    const int grid = std::max(1, std::min(compute_units * per_cu, (nrb + kGemmBlock / 64 - 1) / (kGemmBlock / 64)));
    const int lds = w_bytes + (rows ? (kGemmBlock / 64) * kGemmSeg * 32 * 4 : 0);  // + the wavefronts' row numbers
#define CALL3(NB_, LIST_, G4C_, YPOS_)                                                              \
  err = allow_lds(gemm_rows_kernel<NB_, LIST_, G4C_, YPOS_>, lds);                                  \
  if (err == hipSuccess)                                                                            \
    hipLaunchKernelGGL((gemm_rows_kernel<NB_, LIST_, G4C_, YPOS_>), dim3(grid), dim3(kGemmBlock), lds, st, X, W, Y, \
                       rows, n_rows, K)
  // K = 128 and 256 with up to 128 columns have kernels of their own (K built in)
#define CALL2(NB_, LIST_, YPOS_)                        \
  do {                                                  \
    if constexpr (NB_ <= 4) {                           \
      if (K == 128) { CALL3(NB_, LIST_, 4, YPOS_); }    \
      else if (K == 256) { CALL3(NB_, LIST_, 8, YPOS_); } \
      else { CALL3(NB_, LIST_, 0, YPOS_); }             \
    } else {                                            \
      CALL3(NB_, LIST_, 0, YPOS_);                      \
    }                                                   \
  } while (0)
#define CALL(NB_) do { if (rows && y_by_position) { CALL2(NB_, true, true); } else if (rows) { CALL2(NB_, true, false); } else { CALL2(NB_, false, false); } } while (0)
    TF_DISPATCH_NB(NB, CALL);
#undef CALL
#undef CALL2
#undef CALL3
    return err != hipSuccess ? err : hipGetLastError();
  }
  if (rows) return hipErrorInvalidValue;  // the streamed-W kernel takes contiguous rows only
  const int kc = std::min(K, std::max(8, (32768 / (4 * N)) / 8 * 8));
  const int blocks = (n_rows + 127) / 128;
  const int per = per_xcd_of(blocks);
  const int lds_bytes = kc * N * 4;
#define CALL(NB_)                                                                               \
  err = allow_lds(gemm_kernel<NB_>, lds_bytes);                                                 \
  if (err == hipSuccess)                                                                        \
    hipLaunchKernelGGL((gemm_kernel<NB_>), dim3(grid_of(blocks)), dim3(kBlock), lds_bytes, st, X, W, \
                       Y, n_rows, K, kc, per, blocks)
  TF_DISPATCH_NB(NB, CALL);
#undef CALL
  return err != hipSuccess ? err : hipGetLastError();
}

hipError_t launch_copy_cols(const float *src, int src_rows, int ld_src, int src_col0, int src_cols, float *dst, int rows,
                            int ld_dst, int dst_col0, int cols, int accumulate, hipStream_t st) {
  const size_t n = (size_t)rows * cols;
  if (n == 0) return hipSuccess;
  const int blocks = (int)std::min<size_t>((n + 255) / 256, 65536);
  hipLaunchKernelGGL(copy_cols_kernel, dim3(blocks), dim3(256), 0, st, src, src_rows, ld_src, src_col0, src_cols, dst, rows,
                     ld_dst, dst_col0, cols, accumulate);
  return hipGetLastError();
}

hipError_t launch_pad(const float *src, int src_rows, int ld_src, float *dst, int rows, int ld_dst, hipStream_t st) {
  const size_t n = (size_t)rows * ld_dst;
  if (n == 0) return hipSuccess;
  const int blocks = (int)std::min<size_t>((n + kBlock - 1) / kBlock, 65536);
  hipLaunchKernelGGL(pad_kernel, dim3(blocks), dim3(kBlock), 0, st, src, src_rows, ld_src, dst, rows, ld_dst);
  return hipGetLastError();
}

hipError_t launch_zero_rows(const int *rows, int n_rows, float *Y, int N, hipStream_t st) {
  if (n_rows <= 0) return hipSuccess;
  const size_t units = (size_t)n_rows * (N % 4 == 0 ? N / 4 : N);
  const unsigned blocks = (unsigned)std::min<size_t>((units + 255) / 256, 1u << 20);
  if (N % 4 == 0) hipLaunchKernelGGL((zero_rows_kernel<4>), dim3(blocks), dim3(256), 0, st, rows, units, Y, N);
  else hipLaunchKernelGGL((zero_rows_kernel<1>), dim3(blocks), dim3(256), 0, st, rows, units, Y, N);
  return hipGetLastError();
}

hipError_t launch_relu(float *p, size_t n, hipStream_t st) {
  if (n == 0) return hipSuccess;
  const int blocks = (int)std::max<size_t>(1, std::min<size_t>((n / 4 + 255) / 256, 65536));
  hipLaunchKernelGGL(relu_kernel, dim3(blocks), dim3(256), 0, st, p, n);
  return hipGetLastError();
}

hipError_t launch_xcd_probe(int *out, int n, hipStream_t st) {
  hipLaunchKernelGGL(xcd_probe_kernel, dim3(n), dim3(64), 0, st, out);
  return hipGetLastError();
}

hipError_t launch_fill(float *p, size_t n, float v, hipStream_t st) {
  if (n == 0) return hipSuccess;
  const int blocks = (int)std::min<size_t>((n + 255) / 256, 65536);
  hipLaunchKernelGGL(fill_kernel, dim3(blocks), dim3(256), 0, st, p, n, v);
  return hipGetLastError();
}

hipError_t launch_march_fill(const int *off, const int *src, const float *Ax, const float *Bx, int *ell, size_t n,
                             hipStream_t st) {
  if (n == 0) return hipSuccess;
  const int blocks = (int)std::min<size_t>((n + kBlock - 1) / kBlock, 65536);
  hipLaunchKernelGGL(march_fill_kernel, dim3(blocks), dim3(kBlock), 0, st, off, src, Ax, Bx, reinterpret_cast<int2 *>(ell), n);
  return hipGetLastError();
}

hipError_t launch_fused_spmm_spmm_march(const int *runs, int n_runs, const int *row_ptr, const int *load_ptr,
                                        const int *load_list, const int *row_out, const int *ell, const float *C,
                                        float *D, float *trash, int N, int lds_bytes, int tpg, int dpg, int lpg,
                                        int width, int accumulate, hipStream_t st) {
  if (n_runs <= 0) return hipSuccess;
  // (rows per lane group and iteration beyond what the kernel's register sets hold would be skipped silently)
  if (N % 64 != 0 || tpg < 1 || tpg > kMarchTpg || dpg < 1 || dpg > kMarchDpg || lpg < 1 || lpg > kMarchLpg || lds_bytes > 163840 ||
      width < 0 || width > kMarchWideW)
    return hipErrorInvalidValue;
  const int per = per_xcd_of(n_runs);
  hipError_t err = hipSuccess;
#define CALLM3(ACC_, W_, WIDE_)                                                                                   \
  err = allow_lds(fused_spmm_spmm_march_kernel<ACC_, W_, WIDE_>, lds_bytes);                                      \
  if (err == hipSuccess)                                                                                          \
    hipLaunchKernelGGL((fused_spmm_spmm_march_kernel<ACC_, W_, WIDE_>), dim3(grid_of(n_runs)), dim3(kMarchBlock), \
                       lds_bytes, st, reinterpret_cast<const int2 *>(runs), n_runs, per, row_ptr, load_ptr,       \
                       reinterpret_cast<const int2 *>(load_list), row_out, reinterpret_cast<const int4 *>(ell), C, D, trash, N)
#define CALLM(W_, WIDE_) do { if (accumulate) { CALLM3(true, W_, WIDE_); } else { CALLM3(false, W_, WIDE_); } } while (0)
  if (width <= kMarchW) {  // 64-byte ELL rows, the pairs spread over a quad
    switch (width <= 5 ? 5 : width) {
      case 5: CALLM(5, false); break;
      case 6: CALLM(6, false); break;
      case 7: CALLM(7, false); break;
      default: CALLM(8, false); break;
    }
  } else {  // 256-byte ELL rows, the pairs spread over the lane group: the kernel built for the next width up
    if (width <= 12) CALLM(12, true);
    else if (width <= 16) CALLM(16, true);
    else if (width <= 20) CALLM(20, true);
    else if (width <= 28) CALLM(28, true);
    else CALLM(32, true);
  }
#undef CALLM
#undef CALLM3
  return err != hipSuccess ? err : hipGetLastError();
}

}  // namespace tf
