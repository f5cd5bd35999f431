// Two GCN layers in one tile:  D = A * (act(A * (X * W1)) * W2)  with the hidden layer in LDS.
//
// The reference's fusedGCN walks every tile through four kernels -- GEMM, SpMM, GEMM, SpMM
// (binding-project/src/Functions.cpp:228-290, MixPtr[4j .. 4j+3]) -- so that the first layer's output
// never leaves the cache before the second layer reads it.  Here a tile is one workgroup and the
// cache is its LDS.  A tile owns the rows [o0, o1) of D.  Those read the rows [h0, h1) of the second
// layer's intermediate T2 = Hid * W2, i.e. of the hidden layer Hid; the hidden rows [h0, h1) read the
// rows [t0, t1) of the first layer's intermediate T1 = X * W1.  The tile computes all of them itself
// (rows outside [o0, o1) are halo rows that its neighbours compute too: tiling with redundancy, as in
// fusion/src/SpMM_SpMM.cpp:984-1057), one phase after the other:
//
//   1  T1[t0, t1) = X[t0, t1) * W1      fp32 MFMA, W1 in registers, X through two staging buffers -> slab A
//   2  Hid[h0, h1) = act(A[h0, h1) * T1)  lane groups gather out of slab A                         -> slab B
//   3  T2[h0, h1) = Hid * W2             fp32 MFMA, W2 in registers, Hid read from slab B          -> slab A
//   4  D[o0, o1) = A[o0, o1) * T2        lane groups gather out of slab A                          -> HBM
//
// The rows of A that the two gather phases walk -- one stretch of the CSR arrays, [min(o0, h0), max(o1, h1)) -- are
// copied into LDS at the start of the tile, so that no gather waits for a row pointer or a (column, value) pair
// from memory.  Only X, the weights, A's rows and D cross HBM.
//
// Where a tile's time goes (cycle counter per phase; band of 32, K = H = N = 128: 95 rows owned, 124 hidden rows,
// 154 rows of the first intermediate, 120,000 cycles a tile): weights and A's rows 6 %, phase 1 37 % (its MFMAs
// alone would take 20 %: one barrier per 32 values of k, with both wavefronts of a SIMD waiting for their LDS operands
// at the same time), phase 2 21 %, phase 3 21 % (13 %), phase 4 15 %.  The phases run one after the other and all
// wavefronts are in the same one, so MFMA, LDS and VALU never overlap -- which the streamed kernel's producer and
// consumer wavefronts do all the time; this kernel trades that for keeping the hidden layer out of HBM.  The MFMA phases are the register-W producer of
// fused_gemm_spmm_regw_kernel: v_mfma_f32_16x16x4_f32, a wavefront owns 16 output columns and keeps its
// K x 16 slice of the weight in registers; when the width has fewer than eight column blocks, the
// wavefronts that share a block split the four 16-row blocks of a 64-row step among themselves.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "tf_device.h"

namespace tf {

typedef float g2_v4f __attribute__((ext_vector_type(4)));
constexpr int kG2Block = 512;                       // eight wavefronts
constexpr int kG2Pad = 4;                           // floats between slab rows beyond the width: lanes of a read in different banks
constexpr int kG2XRows = 64, kG2XChunk = 32, kG2XLd = kG2XChunk + 4;
constexpr int kG2StageFloats = 2 * kG2XRows * kG2XLd;  // both staging buffers of X
static_assert(kG2StageFloats == kTile2StageFloats && kG2Pad == kTile2Pad, "the inspector sizes the slabs with these");

// One MFMA phase's share of a 64-row step: acc[bi] += A-operand rows (16 bi + j) x this wavefront's weight slice,
// for the 16-row blocks bi this wavefront takes.  `xrow(bi)` = LDS address of row 16 bi + j, k = 0.
template <int RG, class RowPtr>
__device__ __forceinline__ void g2_mfma_16k(const RowPtr &xrow, int koff, int h, int rg, const float *w, g2_v4f (&acc)[4]) {
  fvec<4> a[4];
#pragma unroll
  for (int bi = 0; bi < 4; ++bi)
    if ((bi % RG) == rg) a[bi] = *reinterpret_cast<const fvec<4> *>(xrow(bi) + koff + 4 * h);
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int bi = 0; bi < 4; ++bi)
      if ((bi % RG) == rg) acc[bi] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[bi].v[u], w[u], acc[bi], 0, 0, 0);
}

template <int KS1, int KS2, int NS>
__global__ __launch_bounds__(kG2Block) void fused_gcn2_kernel(
    const Tile2 *__restrict__ tiles, int n_tiles, int per_xcd, const float *__restrict__ X, const float *__restrict__ W1,
    const float *__restrict__ W2, int K, const int *__restrict__ Ap, const int *__restrict__ Ai,
    const float *__restrict__ Ax, float *__restrict__ D, int relu, int accumulate) {
  static_assert(KS1 % 2 == 0 && (KS2 == 2 || KS2 == 4 || KS2 == 8) && (NS == 2 || NS == 4 || NS == 8), "widths of 32, 64 or 128");
  constexpr int H = 16 * KS2, N = 16 * NS;
  constexpr int LPRH = H / 4, LPRN = N / 4;
  constexpr int ldh = H + kG2Pad, ldn = N + kG2Pad;
  constexpr int RGH = 8 / KS2, RGN = 8 / NS;  // wavefronts per column block
  extern __shared__ __align__(16) float lds[];
  const int tile = xcd_contiguous(blockIdx.x, per_xcd);
  if (tile >= n_tiles) return;
  const Tile2 t = tiles[tile];
  const int P1 = t.t1 - t.t0, PH = t.h1 - t.h0;
  float *slabA = lds;             // T1 (P1 x ldh), later T2 (PH x ldn)
  float *slabB = lds + t.b_off;   // the staging buffers of X, later Hid (PH x ldh)
  // the tile's rows of A: row pointers (relative), columns, values
  const int c0 = PH > 0 ? min(t.o0, t.h0) : t.o0, c1 = PH > 0 ? max(t.o1, t.h1) : t.o1;
  const int kbase = Ap[c0], nC = Ap[c1] - kbase;
  int *rp = reinterpret_cast<int *>(lds + t.c_off);
  int *ci = rp + (c1 - c0 + 1 + 3) / 4 * 4;
  float *cv = reinterpret_cast<float *>(ci + (nC + 3) / 4 * 4);
  for (int x = threadIdx.x; x <= c1 - c0; x += kG2Block) rp[x] = Ap[c0 + x] - kbase;
  for (int x = threadIdx.x; x < nC; x += kG2Block) {
    ci[x] = Ai[kbase + x];
    cv[x] = Ax[kbase + x];
  }
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int j = lane % 16, h = lane / 16;
  const int cbh = wave % KS2, rgh = wave / KS2;
  const int cbn = wave % NS, rgn = wave / NS;

  // staging role of this thread in phase 1: 16 bytes of row sr of every 64 x 32 chunk of X
  const int sr = threadIdx.x / 8, sk = (threadIdx.x % 8) * 4;
  const int nkc = (K + kG2XChunk - 1) / kG2XChunk;
  const int nchunks = ((P1 + kG2XRows - 1) / kG2XRows) * nkc;
  auto chunk_unit = [&](int ch) -> fvec<4> {
    const int q = ch / nkc, k = (ch % nkc) * kG2XChunk + sk;
    const int row = t.t0 + min(q * kG2XRows + sr, P1 - 1);  // rows past the end repeat the last one
    return (ch < nchunks && k < K) ? load4(X + (size_t)row * K + k) : vzero<4>();
  };
  fvec<4> x0 = chunk_unit(0), x1 = chunk_unit(1), x2 = chunk_unit(2);

  // both weight slices: lane (j, h) holds W[16 m + 4 h + u][16 cb + j] in w[4 m + u]
  float w1[KS1 * 4], w2[KS2 * 4];
#pragma unroll
  for (int m = 0; m < KS1; ++m)
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = 16 * m + 4 * h + u;
      w1[4 * m + u] = k < K ? W1[(size_t)k * H + 16 * cbh + j] : 0.f;
    }
#pragma unroll
  for (int m = 0; m < KS2; ++m)
#pragma unroll
    for (int u = 0; u < 4; ++u) w2[4 * m + u] = W2[(size_t)(16 * m + 4 * h + u) * N + 16 * cbn + j];

  // ---- phase 1: T1 = X * W1 --------------------------------------------------------------------
  if (nchunks > 0) *reinterpret_cast<fvec<4> *>(slabB + sr * kG2XLd + sk) = x0;
  x0 = x1;
  x1 = x2;
  __syncthreads();
  int ch = 0;
  for (int r0 = 0; r0 < P1; r0 += kG2XRows) {
    g2_v4f acc[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[b] = g2_v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kc = 0; kc < KS1 / 2; ++kc) {
      if (kc * kG2XChunk < K) {  // uniform
        x2 = chunk_unit(ch + 3);
        const float *xb = slabB + (ch & 1) * (kG2XRows * kG2XLd);
        auto xrow = [&](int bi) { return xb + (16 * bi + j) * kG2XLd; };
        g2_mfma_16k<RGH>(xrow, 0, h, rgh, w1 + 4 * (2 * kc), acc);
        g2_mfma_16k<RGH>(xrow, 16, h, rgh, w1 + 4 * (2 * kc + 1), acc);
        if (ch + 1 < nchunks) *reinterpret_cast<fvec<4> *>(slabB + ((ch + 1) & 1) * (kG2XRows * kG2XLd) + sr * kG2XLd + sk) = x0;
        x0 = x1;
        x1 = x2;
        ++ch;
        lds_barrier();  // (LDS traffic only: the loads of X that are on their way stay on their way)
      }
    }
    // accumulator register r of lane (j, h) is output row 4 h + r, column j of its block
#pragma unroll
    for (int bi = 0; bi < 4; ++bi)
      if ((bi % RGH) == rgh) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int lr = r0 + 16 * bi + 4 * h + r;
          if (lr < P1) slabA[lr * ldh + 16 * cbh + j] = acc[bi][r];
        }
      }
  }
  __syncthreads();  // T1 complete; the staging buffers are free

  // ---- phase 2: Hid = act(A[h0, h1) * T1) ----------------------------------------------------------
  {
    constexpr int G = kG2Block / LPRH;
    const int group = threadIdx.x / LPRH, glane = threadIdx.x % LPRH;
    const LdsRows<4> src{slabA, ldh, glane * 4, t.t0};
    for (int r = t.h0 + group; r < t.h1; r += G) {
      fvec<4> acc = vzero<4>();
      row_dot_direct<4, LPRH>(ci, cv, rp[r - c0], rp[r - c0 + 1], true, src, acc);
      if (relu) {
#pragma unroll
        for (int c = 0; c < 4; ++c) acc.v[c] = fmaxf(acc.v[c], 0.f);
      }
      *reinterpret_cast<fvec<4> *>(slabB + (r - t.h0) * ldh + glane * 4) = acc;
    }
  }
  __syncthreads();  // Hid complete; T1 is dead

  // ---- phase 3: T2 = Hid * W2 ----------------------------------------------------------------------
  for (int r0 = 0; r0 < PH; r0 += 64) {
    g2_v4f acc[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[b] = g2_v4f{0.f, 0.f, 0.f, 0.f};
    auto xrow = [&](int bi) { return slabB + min(r0 + 16 * bi + j, PH - 1) * ldh; };
#pragma unroll
    for (int m = 0; m < KS2; ++m) g2_mfma_16k<RGN>(xrow, 16 * m, h, rgn, w2 + 4 * m, acc);
#pragma unroll
    for (int bi = 0; bi < 4; ++bi)
      if ((bi % RGN) == rgn) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int lr = r0 + 16 * bi + 4 * h + r;
          if (lr < PH) slabA[lr * ldn + 16 * cbn + j] = acc[bi][r];
        }
      }
  }
  __syncthreads();  // T2 complete

  // ---- phase 4: D = A[o0, o1) * T2 -------------------------------------------------------------------
  {
    constexpr int G = kG2Block / LPRN;
    const int group = threadIdx.x / LPRN, glane = threadIdx.x % LPRN;
    const LdsRows<4> src{slabA, ldn, glane * 4, t.h0};
    for (int i = t.o0 + group; i < t.o1; i += G) {
      float *dst = D + (size_t)i * N + glane * 4;
      fvec<4> acc = vzero<4>();
      if (accumulate) acc = *reinterpret_cast<const fvec<4> *>(dst);
      row_dot_direct<4, LPRN>(ci, cv, rp[i - c0], rp[i - c0 + 1], true, src, acc);
      store_streaming<4>(dst, acc);
    }
  }
}

namespace {
template <class F> hipError_t g2_allow_lds(F kernel, int bytes) {
  if (bytes <= 65536) return hipSuccess;
  return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}
}  // namespace

// K: columns of X (a multiple of 8, at most 256); H, N in {32, 64, 128}.  lds_bytes: what the fullest tile needs.  hipErrorInvalidValue for widths the kernel is not built for.
hipError_t launch_fused_gcn2(const Tile2 *tiles, int n_tiles, const float *X, const float *W1, const float *W2, int K, int H,
                             int N, const int *Ap, const int *Ai, const float *Ax, float *D, int lds_bytes,
                             int relu, int accumulate, hipStream_t st) {
  if (n_tiles <= 0) return hipSuccess;
  if (K <= 0 || K > 256 || K % 8 != 0 || (H != 32 && H != 64 && H != 128) || (N != 32 && N != 64 && N != 128)) return hipErrorInvalidValue;
  const int KS1 = K <= 64 ? 4 : K <= 128 ? 8 : 16;
  const int grid = (n_tiles + kXcds - 1) / kXcds * kXcds, per = (n_tiles + kXcds - 1) / kXcds;
  hipError_t err = hipSuccess;
#define G2_CALL(KS1_, KS2_, NS_)                                                                                          \
  do {                                                                                                                    \
    err = g2_allow_lds(fused_gcn2_kernel<KS1_, KS2_, NS_>, lds_bytes);                                                    \
    if (err == hipSuccess)                                                                                                \
      hipLaunchKernelGGL((fused_gcn2_kernel<KS1_, KS2_, NS_>), dim3(grid), dim3(kG2Block), lds_bytes, st, tiles, n_tiles, \
                         per, X, W1, W2, K, Ap, Ai, Ax, D, relu, accumulate);                                          \
  } while (0)
#define G2_N(KS1_, KS2_) do { if (N == 32) G2_CALL(KS1_, KS2_, 2); else if (N == 64) G2_CALL(KS1_, KS2_, 4); else G2_CALL(KS1_, KS2_, 8); } while (0)
#define G2_H(KS1_) do { if (H == 32) G2_N(KS1_, 2); else if (H == 64) G2_N(KS1_, 4); else G2_N(KS1_, 8); } while (0)
  if (KS1 == 4) G2_H(4); else if (KS1 == 8) G2_H(8); else G2_H(16);
#undef G2_H
#undef G2_N
#undef G2_CALL
  return err != hipSuccess ? err : hipGetLastError();
}

}  // namespace tf
