/*
 * tf_oracle.c -- CPU restatement of tile-fusion's fused executors and inspectors.
 *
 * THIS IS TEST INFRASTRUCTURE.  It is the checker the HIP library is compared
 * against (tests, the smoke check, the CPU-baseline leg of the benchmark).  The
 * product library never links, loads or calls anything in this file.
 *
 * Every function cites the reference file:line (relative to the reference
 * checkout) whose algorithm it restates.  Arithmetic is fp32 with fused
 * multiply-add in CSR order, which is what the reference's AVX2 kernels do.
 *
 * Pinning status (what independent evidence holds each function in place):
 *   orc_spmm_csr, orc_spmm_spmm_fused, orc_spmm_spmm_fused_separated:
 *       bitwise against the reference's own translation units compiled in
 *       place (oracle/_ref), float64 scipy products, integer closed forms on
 *       Laplacians, brute force on tiny inputs.                         PINNED
 *   orc_gemm_spmm_fused:  float64 numpy/scipy product, A=I / C=I reductions,
 *       integer-valued inputs (exact in fp32).  The reference's GEMM is Intel
 *       MKL cblas_sgemm, which is not in the reference tree: the bit pattern of
 *       its result is PARITY UNPINNED (tolerance only); sgemm here is the
 *       textbook row-major product.
 *   orc_inspect_vt_gemm_spmm, orc_inspect_vt_both_wavefronts,
 *   orc_inspect_fixed_tiles:  the reference inspectors need un-vendored
 *       headers and cannot be compiled; they are pinned by schedule
 *       invariants, hand-derived schedules for banded matrices and the
 *       closed-form tile counts of the halving rule.  The exact array contents
 *       for arbitrary matrices are PARITY UNPINNED beyond those cases.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_OK 0
#define ORC_EINVAL (-1)
#define ORC_ENOTERM (-2) /* the reference loop would not terminate on this input */
#define ORC_ENOMEM (-3)

/* Flat two-level schedule, the layout of sym_lib::MultiDimensionalSet
 * (fusion/include/sparse-fusion/MultiDimensionalSet.h:15-21). */
typedef struct {
  int n1;         /* number of levels (2)                         n1_        */
  int n_part;     /* ptr1[n1]                                                */
  int n_id;       /* ptr2[n_part]                                            */
  int *ptr1;      /* [n1+1]      level -> partition range         ptr1_      */
  int *ptr2;      /* [n_part+1]  partition -> id range            ptr2_      */
  int *ker_begin; /* [2*n_part]  end of op-0 ids, end of op-1 ids ker_begin_ */
  int *id;        /* [n_id]      row ids                          id_        */
  int *type;      /* [n_id]      0 = first op, 1 = second op      type_      */
} orc_schedule;

void orc_schedule_free(orc_schedule *s) {
  if (!s) return;
  free(s->ptr1); free(s->ptr2); free(s->ker_begin); free(s->id); free(s->type);
  memset(s, 0, sizeof(*s));
}

/* ------------------------------------------------------------------------ */
/* Executors                                                                 */
/* ------------------------------------------------------------------------ */

/* One CSR row times a dense row-major matrix, accumulated into out[0..N):
 * out[c] = fma(Ax[j], X[Ai[j]*N + c], out[c]) for j in CSR order.
 * Same per-element operation sequence as the AVX2 kernels
 * (fusion/src/SpMM_SpMM_vectorized.cpp:892-936: load, fmadd per nnz, store). */
static inline void row_axpy(const int *Ap, const int *Ai, const float *Ax, int i,
                            const float *X, int N, float *out) {
  for (int j = Ap[i]; j < Ap[i + 1]; ++j) {
    const float a = Ax[j];
    const float *x = X + (size_t)Ai[j] * N;
    for (int c = 0; c < N; ++c) out[c] = fmaf(a, x[c], out[c]);
  }
}

/* Cx += A * Bx.  fusion/src/SpMM_SpMM.cpp:20-31 (sequential) and :37-55
 * (parallel over rows).  Cx is accumulated into, as in the reference. */
void orc_spmm_csr(int M, int N, const int *Ap, const int *Ai, const float *Ax,
                  const float *Bx, float *Cx, int nthreads) {
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (int i = 0; i < M; ++i) row_axpy(Ap, Ai, Ax, i, Bx, N, Cx + (size_t)i * N);
}

/* D += B * (A * C) over an interleaved (id,type) schedule.
 * fusion/src/SpMM_SpMM.cpp:211-248 (scalar) and
 * fusion/src/SpMM_SpMM_vectorized.cpp:876-989 (AVX2, same FMA sequence).
 * Argument names follow the reference: (Ap,Ai,Ax) is the inner sparse matrix
 * applied to dense Cx giving ACx; (Bp,Bi,Bx) is the outer one giving Dx.
 * ACx and Dx must be zero on entry. */
void orc_spmm_spmm_fused(int M, int N, const int *Ap, const int *Ai, const float *Ax,
                         const int *Bp, const int *Bi, const float *Bx,
                         const float *Cx, float *Dx, float *ACx, int LevelNo,
                         const int *LevelPtr, const int *ParPtr, const int *Partition,
                         const int *ParType, int nthreads) {
  (void)M;
  for (int l = 0; l < LevelNo; ++l) {
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int p = LevelPtr[l]; p < LevelPtr[l + 1]; ++p) {
      for (int k = ParPtr[p]; k < ParPtr[p + 1]; ++k) {
        const int i = Partition[k];
        if (ParType[k] == 0)
          row_axpy(Ap, Ai, Ax, i, Cx, N, ACx + (size_t)i * N);
        else
          row_axpy(Bp, Bi, Bx, i, ACx, N, Dx + (size_t)i * N);
      }
    }
  }
}

/* Same product over the "separated" schedule walk: a partition's first-op rows
 * are the contiguous range starting at Partition[ParPtr[p]] of length
 * MixPtr[2p]-ParPtr[p]; its second-op ids are [MixPtr[2p], MixPtr[2p+1]).
 * fusion/src/SpMM_SpMM_vectorized.cpp:993-1110 (one sparse matrix for both). */
void orc_spmm_spmm_fused_separated(int M, int N, const int *Ap, const int *Ai,
                                   const float *Ax, const float *Cx, float *Dx,
                                   float *ACx, int LevelNo, const int *LevelPtr,
                                   const int *ParPtr, const int *Partition,
                                   const int *MixPtr, int nthreads) {
  (void)M;
  for (int l = 0; l < LevelNo; ++l) {
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int p = LevelPtr[l]; p < LevelPtr[l + 1]; ++p) {
      const int kb = ParPtr[p], ke1 = MixPtr[2 * p], ke2 = MixPtr[2 * p + 1];
      const int tile = ke1 - kb;
      if (tile > 0) {
        const int i0 = Partition[kb];
        for (int i = i0; i < i0 + tile; ++i)
          row_axpy(Ap, Ai, Ax, i, Cx, N, ACx + (size_t)i * N);
      }
      for (int k = ke1; k < ke2; ++k) {
        const int i = Partition[k];
        row_axpy(Ap, Ai, Ax, i, ACx, N, Dx + (size_t)i * N);
      }
    }
  }
}

/* Row-major out[T x N] = X[T x K] * W[K x N], beta = 0: the call
 * cblas_sgemm(RowMajor, NoTrans, NoTrans, T, N, K, 1, X, K, W, N, 0, out, N)
 * at fusion/gcn/GCN_Layer_MKL_Forward_Utils.h:233-237.  Textbook product:
 * every element is one chain of fused multiply-adds with k ascending; MKL's
 * internal order is not reproducible (see header).
 *
 * Two bodies with the same arithmetic per element, hence the same bits:
 *   sgemm_rows_scalar   4 x 32 blocks of plain fmaf (what -march=x86-64-v3 makes
 *                       of it: AVX2), any shape;
 *   sgemm_rows_avx512   register-blocked micro-kernel for hosts with AVX-512
 *                       (checked at run time): 8 rows x 32 columns of
 *                       accumulators in 16 zmm registers, per k two loads of W
 *                       and eight broadcasts of X; the column block is the outer
 *                       loop so that its 32-column panel of W stays in L1 for
 *                       all row blocks of the tile.  This is the class of
 *                       kernel the reference gets from MKL, so that the CPU
 *                       baseline built on it is one worth standing next to. */
static void sgemm_rows_scalar(int T, int N, int K, const float *X, const float *W, float *out, int j_begin) {
  enum { RB = 4, CB = 32 };
  for (int i0 = 0; i0 < T; i0 += RB) {
    const int rb = (T - i0 < RB) ? (T - i0) : RB;
    for (int j0 = j_begin; j0 < N; j0 += CB) {
      const int cb = (N - j0 < CB) ? (N - j0) : CB;
      float acc[RB][CB];
      for (int r = 0; r < RB; ++r)
        for (int c = 0; c < CB; ++c) acc[r][c] = 0.0f;
      if (rb == RB && cb == CB) {
        for (int k = 0; k < K; ++k) {
          const float *w = W + (size_t)k * N + j0;
          for (int r = 0; r < RB; ++r) {
            const float a = X[(size_t)(i0 + r) * K + k];
            for (int c = 0; c < CB; ++c) acc[r][c] = fmaf(a, w[c], acc[r][c]);
          }
        }
      } else {
        for (int k = 0; k < K; ++k) {
          const float *w = W + (size_t)k * N + j0;
          for (int r = 0; r < rb; ++r) {
            const float a = X[(size_t)(i0 + r) * K + k];
            for (int c = 0; c < cb; ++c) acc[r][c] = fmaf(a, w[c], acc[r][c]);
          }
        }
      }
      for (int r = 0; r < rb; ++r)
        for (int c = 0; c < cb; ++c) out[(size_t)(i0 + r) * N + j0 + c] = acc[r][c];
    }
  }
}

#if defined(__x86_64__)
#include <immintrin.h>
#define ORC_HAVE_AVX512_BODY 1
/* rows [0, T8) (T8 a multiple of 8) x columns [0, N32) (a multiple of 32) */
__attribute__((target("avx512f"))) static void sgemm_rows_avx512(int T8, int N32, int N, int K, const float *X,
                                                                  const float *W, float *out) {
  for (int j0 = 0; j0 < N32; j0 += 32) {
    for (int i0 = 0; i0 < T8; i0 += 8) {
      __m512 a0[8], a1[8];
      for (int r = 0; r < 8; ++r) { a0[r] = _mm512_setzero_ps(); a1[r] = _mm512_setzero_ps(); }
      const float *x = X + (size_t)i0 * K;
      const float *w = W + j0;
      for (int k = 0; k < K; ++k) {
        const __m512 w0 = _mm512_loadu_ps(w + (size_t)k * N);
        const __m512 w1 = _mm512_loadu_ps(w + (size_t)k * N + 16);
#pragma GCC unroll 8
        for (int r = 0; r < 8; ++r) {
          const __m512 xv = _mm512_set1_ps(x[(size_t)r * K + k]);
          a0[r] = _mm512_fmadd_ps(xv, w0, a0[r]);
          a1[r] = _mm512_fmadd_ps(xv, w1, a1[r]);
        }
      }
      for (int r = 0; r < 8; ++r) {
        _mm512_storeu_ps(out + (size_t)(i0 + r) * N + j0, a0[r]);
        _mm512_storeu_ps(out + (size_t)(i0 + r) * N + j0 + 16, a1[r]);
      }
    }
  }
}
#else
#define ORC_HAVE_AVX512_BODY 0
#endif

static int g_simd = -1; /* -1: not decided yet; 0: scalar body only; 1: AVX-512 body where it applies */

/* 1 when the AVX-512 body is in use.  orc_set_simd(0) forces the scalar body (tests compare the two). */
int orc_simd(void) {
  if (g_simd < 0) {
#if ORC_HAVE_AVX512_BODY
    g_simd = __builtin_cpu_supports("avx512f") ? 1 : 0;
#else
    g_simd = 0;
#endif
  }
  return g_simd;
}
void orc_set_simd(int on) {
  g_simd = -1;
  if (!on || !orc_simd()) g_simd = 0;
}

static void sgemm_rows(int T, int N, int K, const float *X, const float *W, float *out) {
#if ORC_HAVE_AVX512_BODY
  if (orc_simd()) {
    const int T8 = T / 8 * 8, N32 = N / 32 * 32;
    if (T8 > 0 && N32 > 0) sgemm_rows_avx512(T8, N32, N, K, X, W, out);
    if (T8 > 0 && N32 < N) sgemm_rows_scalar(T8, N, K, X, W, out, N32);                  /* columns behind the last 32 */
    if (T8 < T) sgemm_rows_scalar(T - T8, N, K, X + (size_t)T8 * K, W, out + (size_t)T8 * N, 0); /* rows behind the last 8 */
    return;
  }
#endif
  sgemm_rows_scalar(T, N, K, X, W, out, 0);
}

/* out = X * W for the whole matrix (the unfused baseline's GEMM,
 * fusion/gcn/GCN_Layer_MKL_Forward_Utils.h:1144), row blocks in parallel. */
void orc_sgemm(int M, int N, int K, const float *X, const float *W, float *out,
               int nthreads) {
  const int blk = 64;
  const int nb = (M + blk - 1) / blk;
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (int b = 0; b < nb; ++b) {
    const int i0 = b * blk;
    const int t = (M - i0 < blk) ? (M - i0) : blk;
    sgemm_rows(t, N, K, X + (size_t)i0 * K, W, out + (size_t)i0 * N);
  }
}

/* Output += A * (Features * Weight), fused over the separated schedule.
 * fusion/gcn/GCN_Layer_MKL_Forward_Utils.h:218-291 (vectorised) and :182-216
 * (scalar twin).  Features is M x K, Weight is K x N (NoTrans, the README's
 * D = A*B*C), Intermediate is M x N scratch, Output must be zero on entry.
 * Unlike the reference, N need not be a multiple of 32. */
void orc_gemm_spmm_fused(int M, const int *Ap, const int *Ai, const float *Ax, int K,
                         int N, const float *Features, const float *Weight,
                         float *Output, float *Intermediate, int nthreads, int LevelNo,
                         const int *LevelPtr, const int *ParPtr, const int *MixPtr,
                         const int *Partition) {
  (void)M;
  for (int l = 0; l < LevelNo; ++l) {
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int p = LevelPtr[l]; p < LevelPtr[l + 1]; ++p) {
      const int kb = ParPtr[p], ke1 = MixPtr[2 * p], ke2 = MixPtr[2 * p + 1];
      const int tile = ke1 - kb;
      if (tile > 0) {
        const int i0 = Partition[kb];
        sgemm_rows(tile, N, K, Features + (size_t)i0 * K, Weight,
                   Intermediate + (size_t)i0 * N);
      }
      for (int k = ke1; k < ke2; ++k) {
        const int i = Partition[k];
        row_axpy(Ap, Ai, Ax, i, Intermediate, N, Output + (size_t)i * N);
      }
    }
  }
}

/* ------------------------------------------------------------------------ */
/* Inspectors                                                                */
/* ------------------------------------------------------------------------ */

typedef struct { int *v; int n, cap; } ivec;
static int iv_push(ivec *a, int x) {
  if (a->n == a->cap) {
    int nc = a->cap ? a->cap * 2 : 64;
    int *nv = (int *)realloc(a->v, (size_t)nc * sizeof(int));
    if (!nv) return -1;
    a->v = nv; a->cap = nc;
  }
  a->v[a->n++] = x;
  return 0;
}

typedef struct { int start, end; int *fused; int nfused; } vtile;
typedef struct { vtile *v; int n, cap; } tvec;
static int tv_push(tvec *a, vtile t) {
  if (a->n == a->cap) {
    int nc = a->cap ? a->cap * 2 : 64;
    vtile *nv = (vtile *)realloc(a->v, (size_t)nc * sizeof(vtile));
    if (!nv) return -1;
    a->v = nv; a->cap = nc;
  }
  a->v[a->n++] = t;
  return 0;
}
static void tv_free(tvec *a) {
  for (int i = 0; i < a->n; ++i) free(a->v[i].fused);
  free(a->v); a->v = 0; a->n = a->cap = 0;
}

static int cmp_int(const void *a, const void *b) {
  int x = *(const int *)a, y = *(const int *)b;
  return (x > y) - (x < y);
}

/* The reference tests a row for fusion by its first and last stored column
 * only (Fusion_Inspector.h:713, :886), i.e. it assumes sorted columns, and it
 * reads outside the row when the row is empty.  Here an empty row counts as
 * fused (it has no dependence at all). */
static inline int row_first(const int *Ap, const int *Ai, int i) { return Ai[Ap[i]]; }
static inline int row_last(const int *Ap, const int *Ai, int i) { return Ai[Ap[i + 1] - 1]; }
static inline int row_empty(const int *Ap, int i) { return Ap[i + 1] == Ap[i]; }

/* Fusion_Inspector.h:1020-1022 */
static int ws_spmm(int nnz, int ucols, int bcol, int tile, int fused, int ds) {
  return (nnz + ucols * bcol + tile * bcol + fused * bcol) * ds + nnz * 4;
}
/* Fusion_Inspector.h:1025-1027 */
static int ws_gemm(int fnnz, int bcol, int ccol, int tile, int fused, int ds) {
  return (tile * ccol + ccol * bcol + tile * bcol + fused * ccol + fnnz) * ds + fnnz * 4;
}
/* Fusion_Inspector.h:1029-1031 */
static int initial_tile_gemm(int bcol, int ccol, int maxws, int ds) {
  return (maxws / ds - bcol * ccol) / (bcol + ccol);
}

/* Initial equal tiles with the remainder rows spread over the leading tiles
 * (Fusion_Inspector.h:857-877 / :683-704), then each row of a tile is fused
 * iff its first and last column fall inside the tile (:883-892 / :710-719). */
static int make_initial_tiles(int M, const int *Ap, const int *Ai, int initial,
                              tvec *tiles, ivec *unfused) {
  const int extra = M % initial;
  const int ntiles = M / initial;
  const int extra_per = (int)ceil(extra / (double)ntiles);
  int removed = 0;
  for (int t = 0; t < ntiles; ++t) {
    vtile vt;
    vt.start = initial * t + removed;
    vt.end = vt.start + initial;
    if (extra > removed) {
      int ext = extra - removed < extra_per ? extra - removed : extra_per;
      vt.end += ext;
      removed += ext;
    }
    vt.fused = (int *)malloc((size_t)(vt.end - vt.start + 1) * sizeof(int));
    vt.nfused = 0;
    if (!vt.fused) return ORC_ENOMEM;
    for (int i = vt.start; i < vt.end; ++i) {
      if (row_empty(Ap, i) || (row_first(Ap, Ai, i) >= vt.start && row_last(Ap, Ai, i) < vt.end))
        vt.fused[vt.nfused++] = i;
      else if (iv_push(unfused, i)) return ORC_ENOMEM;
    }
    if (tv_push(tiles, vt)) return ORC_ENOMEM;
  }
  return ORC_OK;
}

typedef struct {
  int M; const int *Ap; const int *Ai;
  int bcol, ccol, cache, ds;
  int gemm;          /* 1: GeMM-SpMM working set, 0: SpMM-SpMM working set */
  int *stamp; int gen; /* unique-column counting (replaces std::set)      */
  tvec *out; ivec *unfused;
} split_ctx;

static int count_unique_cols(split_ctx *c, int s, int e) {
  int u = 0;
  c->gen++;
  for (int j = c->Ap[s]; j < c->Ap[e]; ++j) {
    int col = c->Ai[j];
    if (c->stamp[col] != c->gen) { c->stamp[col] = c->gen; ++u; }
  }
  return u;
}

/* Tile halving (Fusion_Inspector.h:894-923 / :721-753).  The reference walks a
 * linked list and, after a split, re-examines the left half first; that is a
 * depth-first traversal, written here as recursion.  Takes ownership of
 * t.fused. */
static int split_tile(split_ctx *c, vtile t) {
  const int tile = t.end - t.start;
  int ws;
  if (c->gemm) {
    int fnnz = 0;
    for (int q = 0; q < t.nfused; ++q) fnnz += c->Ap[t.fused[q] + 1] - c->Ap[t.fused[q]];
    ws = ws_gemm(fnnz, c->bcol, c->ccol, tile, t.nfused, c->ds);
  } else {
    int nnz = c->Ap[t.end] - c->Ap[t.start];
    int ucols = count_unique_cols(c, t.start, t.end);
    ws = ws_spmm(nnz, ucols, c->bcol, tile, t.nfused, c->ds);
  }
  if (!(ws > c->cache && tile > 1)) return tv_push(c->out, t) ? ORC_ENOMEM : ORC_OK;
  const int sep = tile / 2 + t.start;
  vtile a, b;
  a.start = t.start; a.end = sep; a.nfused = 0;
  b.start = sep; b.end = t.end; b.nfused = 0;
  a.fused = (int *)malloc((size_t)(t.nfused + 1) * sizeof(int));
  b.fused = (int *)malloc((size_t)(t.nfused + 1) * sizeof(int));
  if (!a.fused || !b.fused) return ORC_ENOMEM;
  for (int q = 0; q < t.nfused; ++q) {
    const int fi = t.fused[q];
    if (row_empty(c->Ap, fi)) { /* no dependence: stays with the half that holds it */
      if (fi < sep) a.fused[a.nfused++] = fi; else b.fused[b.nfused++] = fi;
    } else if (row_last(c->Ap, c->Ai, fi) < sep) a.fused[a.nfused++] = fi;
    else if (row_first(c->Ap, c->Ai, fi) >= sep) b.fused[b.nfused++] = fi;
    else if (iv_push(c->unfused, fi)) return ORC_ENOMEM;
  }
  free(t.fused);
  int rc = split_tile(c, a);
  if (rc) return rc;
  return split_tile(c, b);
}

/* Flatten tiles + remainder partitions into the MultiDimensionalSet layout
 * (Fusion_Inspector.h:959-1010 / :789-840). */
static int emit_schedule(int M, const tvec *tiles, const ivec *unfused, const ivec *ufptr,
                         orc_schedule *S) {
  const int nt = tiles->n, nu = ufptr->n - 1, P = nt + nu;
  memset(S, 0, sizeof(*S));
  S->n1 = 2;
  S->ptr1 = (int *)malloc(3 * sizeof(int));
  S->ptr2 = (int *)malloc((size_t)(P + 1) * sizeof(int));
  S->ker_begin = (int *)malloc((size_t)(2 * P + 1) * sizeof(int));
  S->id = (int *)malloc((size_t)(2 * M + 1) * sizeof(int));
  S->type = (int *)malloc((size_t)(2 * M + 1) * sizeof(int));
  if (!S->ptr1 || !S->ptr2 || !S->ker_begin || !S->id || !S->type) return ORC_ENOMEM;
  S->ptr1[0] = 0; S->ptr1[1] = nt; S->ptr1[2] = P;
  S->ptr2[0] = 0;
  int cnt = 0;
  for (int p = 0; p < nt; ++p) {
    const vtile *t = &tiles->v[p];
    for (int j = t->start; j < t->end; ++j) { S->id[cnt] = j; S->type[cnt] = 0; ++cnt; }
    S->ker_begin[2 * p] = cnt;
    for (int q = 0; q < t->nfused; ++q) { S->id[cnt] = t->fused[q]; S->type[cnt] = 1; ++cnt; }
    S->ker_begin[2 * p + 1] = cnt;
    S->ptr2[p + 1] = cnt;
  }
  for (int p = nt; p < P; ++p) {
    const int u = p - nt;
    S->ker_begin[2 * p] = cnt;
    for (int j = ufptr->v[u]; j < ufptr->v[u + 1]; ++j) {
      S->id[cnt] = unfused->v[j]; S->type[cnt] = 1; ++cnt;
    }
    S->ker_begin[2 * p + 1] = cnt;
    S->ptr2[p + 1] = cnt;
  }
  S->n_part = P;
  S->n_id = cnt;
  return ORC_OK;
}

/* Greedy packing of the sorted unfused rows into remainder partitions in
 * strides that start at 16 rows (Fusion_Inspector.h:924-957 for GeMM-SpMM,
 * :754-787 for SpMM-SpMM).  `both` selects the SpMM-SpMM acceptance test
 * (:770), which also bounds a partition by minMaxTile rows.  The reference's
 * loop does not terminate once its stride has halved to zero; that input is
 * reported as ORC_ENOTERM instead. */
static int pack_unfused(split_ctx *c, const ivec *unfused, int both, int minMaxTile,
                        ivec *ufptr) {
  int stride = 16, nnz = 0, uft = 0, uftile = 0, ucols = 0;
  const int n = unfused->n;
  c->gen++;
  if (iv_push(ufptr, 0)) return ORC_ENOMEM;
  while (uft < n) {
    if (stride <= 0) return ORC_ENOTERM;
    const int lim = (n < uft + stride) ? n : uft + stride;
    for (int ii = uft; ii < lim; ++ii) {
      const int row = unfused->v[ii];
      for (int j = c->Ap[row]; j < c->Ap[row + 1]; ++j) {
        int col = c->Ai[j];
        if (c->stamp[col] != c->gen) { c->stamp[col] = c->gen; ++ucols; }
      }
      nnz += c->Ap[row + 1] - c->Ap[row];
      uftile += 1;
    }
    const int ws = ws_spmm(nnz, ucols, c->bcol, uftile, 0, c->ds);
    int accept;
    if (both) accept = ((ws < c->cache) || (uftile == 1)) && (uftile + stride < minMaxTile);
    else accept = (ws < c->cache) || (uftile <= 16);
    if (accept) {
      uft += stride;
    } else {
      if (iv_push(ufptr, uft)) return ORC_ENOMEM;
      nnz = 0; ucols = 0; c->gen++;
      if (uftile <= stride) stride = stride / 2;
      if (uftile >= 3 * stride) stride = stride * 2;
      uftile = 0;
    }
  }
  if (iv_push(ufptr, n)) return ORC_ENOMEM;
  return ORC_OK;
}

static int inspect_vt(int M, int ncols, const int *Ap, const int *Ai, int bcol, int ccol,
                      int cache, int ds, int gemm, int nthreads, orc_schedule *S) {
  if (M <= 0 || !Ap || !S) return ORC_EINVAL;
  int initial, minMaxTile = 0;
  if (gemm) {
    initial = initial_tile_gemm(bcol, ccol, cache, ds);       /* :856 */
    if (initial > M) initial = M;                              /* :857 */
  } else {
    minMaxTile = M / (2 * nthreads);                           /* :682 */
    initial = 4096 < minMaxTile ? 4096 : minMaxTile;           /* :681-683 */
  }
  if (initial <= 0) return ORC_EINVAL; /* the reference divides by it */
  tvec first = {0, 0, 0}, tiles = {0, 0, 0};
  ivec unfused = {0, 0, 0}, ufptr = {0, 0, 0};
  split_ctx c;
  memset(&c, 0, sizeof(c));
  c.M = M; c.Ap = Ap; c.Ai = Ai; c.bcol = bcol; c.ccol = ccol; c.cache = cache; c.ds = ds;
  c.gemm = gemm; c.out = &tiles; c.unfused = &unfused;
  c.stamp = (int *)calloc((size_t)(ncols > M ? ncols : M) + 1, sizeof(int));
  int rc = c.stamp ? ORC_OK : ORC_ENOMEM;
  if (!rc) rc = make_initial_tiles(M, Ap, Ai, initial, &first, &unfused);
  for (int t = 0; !rc && t < first.n; ++t) {
    vtile vt = first.v[t];
    first.v[t].fused = 0; /* ownership moves to split_tile */
    rc = split_tile(&c, vt);
  }
  if (!rc) {
    qsort(unfused.v, (size_t)unfused.n, sizeof(int), cmp_int); /* :924 / :754 */
    rc = pack_unfused(&c, &unfused, !gemm, minMaxTile, &ufptr);
  }
  if (!rc) rc = emit_schedule(M, &tiles, &unfused, &ufptr, S);
  if (rc) orc_schedule_free(S);
  tv_free(&first); tv_free(&tiles);
  free(unfused.v); free(ufptr.v); free(c.stamp);
  return rc;
}

/* InspectorForTileFusedCSRVariableTileSize::generateVariableTileSizeScheduleGeMMSpMM
 * (Fusion_Inspector.h:850-1017).  BCol = inner dense dimension K, CCol = output
 * columns N, cache = ScheduleParameters::TileM in bytes, DataSize = 4 for fp32. */
int orc_inspect_vt_gemm_spmm(int M, int ncols, const int *Ap, const int *Ai, int BCol,
                             int CCol, int cacheBytes, int DataSize, orc_schedule *S) {
  return inspect_vt(M, ncols, Ap, Ai, BCol, CCol, cacheBytes, DataSize, 1, 1, S);
}

/* ...::generateVariableTileSizeScheduleForBothWavefronts (Fusion_Inspector.h:676-846). */
int orc_inspect_vt_both_wavefronts(int M, int ncols, const int *Ap, const int *Ai, int BCol,
                                   int cacheBytes, int DataSize, int NumThreads,
                                   orc_schedule *S) {
  if (NumThreads <= 0) return ORC_EINVAL;
  return inspect_vt(M, ncols, Ap, Ai, BCol, 0, cacheBytes, DataSize, 0, NumThreads, S);
}

/* partitionByWeight with unit weights (fusion/src/Fusion_Utils.cpp:365-388):
 * each part takes elements until its weight reaches ceil(n / nparts). */
static void partition_unit(int n, int nparts, int *idx /* [nparts+1] */) {
  const double even = ceil((double)n / nparts);
  int j = 0;
  idx[0] = 0;
  for (int p = 0; p < nparts; ++p) {
    double w = 0;
    while (w < even && j < n) { w += 1.0; ++j; }
    idx[p + 1] = j;
  }
}

/* Fixed-size tiles: SparseFusionInspector::generateFusedScheduleForAllFused
 * (Fusion_Inspector.h:32-55) -> SparseFusion::fuse/pairing
 * (fusion/src/SparseFusion.cpp:30-142) with the consecutive seed partitioning
 * of LBC (fusion/src/Fusion_Utils.cpp:510-522) and forward_pairing (:316-350),
 * flattened as MultiDimensionalSet(list, Separated)
 * (fusion/src/MultiDimensionalSet.cpp:124-185).
 * nParts = max(M / IterPerPartition, 2 * NumThreads); a second-op row is
 * fused into the tile that holds it iff every stored column of the row is a
 * row of that tile; the remaining rows are split evenly into nParts
 * partitions of a second level. */
int orc_inspect_fixed_tiles(int M, const int *Ap, const int *Ai, int IterPerPartition,
                            int NumThreads, orc_schedule *S) {
  if (M <= 0 || IterPerPartition <= 0 || NumThreads <= 0 || !S) return ORC_EINVAL;
  int nparts = M / IterPerPartition;
  if (nparts < 2 * NumThreads) nparts = 2 * NumThreads;
  int *tp = (int *)malloc((size_t)(nparts + 1) * sizeof(int));
  int *up = (int *)malloc((size_t)(nparts + 1) * sizeof(int));
  int *unf = (int *)malloc((size_t)(M + 1) * sizeof(int));
  memset(S, 0, sizeof(*S));
  S->n1 = 2;
  S->ptr1 = (int *)malloc(3 * sizeof(int));
  S->ptr2 = (int *)malloc((size_t)(2 * nparts + 1) * sizeof(int));
  S->ker_begin = (int *)malloc((size_t)(4 * nparts + 1) * sizeof(int));
  S->id = (int *)malloc((size_t)(2 * M + 1) * sizeof(int));
  S->type = (int *)malloc((size_t)(2 * M + 1) * sizeof(int));
  if (!tp || !up || !unf || !S->ptr1 || !S->ptr2 || !S->ker_begin || !S->id || !S->type) {
    free(tp); free(up); free(unf); orc_schedule_free(S);
    return ORC_ENOMEM;
  }
  partition_unit(M, nparts, tp);
  int cnt = 0, nunf = 0;
  S->ptr2[0] = 0;
  for (int p = 0; p < nparts; ++p) {
    const int s = tp[p], e = tp[p + 1];
    for (int i = s; i < e; ++i) { S->id[cnt] = i; S->type[cnt] = 0; ++cnt; }
    S->ker_begin[2 * p] = cnt;
    for (int i = s; i < e; ++i) {
      int ok = 1;
      for (int j = Ap[i]; j < Ap[i + 1]; ++j)
        if (Ai[j] < s || Ai[j] >= e) { ok = 0; break; }
      if (ok) { S->id[cnt] = i; S->type[cnt] = 1; ++cnt; } else unf[nunf++] = i;
    }
    S->ker_begin[2 * p + 1] = cnt;
    S->ptr2[p + 1] = cnt;
  }
  int P = nparts;
  if (nunf > 0) { /* SparseFusion.cpp:112-130: a second level only if rows remain */
    partition_unit(nunf, nparts, up);
    for (int q = 0; q < nparts; ++q) {
      S->ker_begin[2 * P] = cnt;
      for (int j = up[q]; j < up[q + 1]; ++j) { S->id[cnt] = unf[j]; S->type[cnt] = 1; ++cnt; }
      S->ker_begin[2 * P + 1] = cnt;
      S->ptr2[P + 1] = cnt;
      ++P;
    }
  }
  S->n1 = (nunf > 0) ? 2 : 1;
  S->ptr1[0] = 0; S->ptr1[1] = nparts; S->ptr1[2] = P;
  S->n_part = P; S->n_id = cnt;
  free(tp); free(up); free(unf);
  return ORC_OK;
}

/* MultiDimensionalSet::getNumberOfFusedNodes / getFusedNnzNum
 * (fusion/src/MultiDimensionalSet.cpp:240-267): second-op ids of level 0. */
void orc_schedule_fused_stats(const orc_schedule *S, const int *Ap, int *fusedNodes,
                              int *fusedNnz) {
  int fn = 0, fz = 0;
  for (int p = S->ptr1[0]; p < S->ptr1[1]; ++p)
    for (int k = S->ptr2[p]; k < S->ptr2[p + 1]; ++k)
      if (S->type[k] == 1) { ++fn; fz += Ap[S->id[k] + 1] - Ap[S->id[k]]; }
  if (fusedNodes) *fusedNodes = fn;
  if (fusedNnz) *fusedNnz = fz;
}

int orc_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
