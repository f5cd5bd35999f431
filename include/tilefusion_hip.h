/*
 * tilefusion_hip.h -- C ABI of libtilefusion_hip, the MI355X (gfx950) engine behind
 * the tile-fusion API (include/tile-fusion.h).
 *
 * Plain pointers, sizes and opaque handles only.  fp32 values, int32 indices, CSR
 * sparse matrices, row-major dense matrices -- the reference's conventions.
 *
 * Each entry point cites the reference interface it stands in for (paths relative
 * to the reference checkout).  Names in the comments follow the README API:
 *     D = A * (B * C)        A sparse;  B sparse (SpMM-SpMM) or dense (GeMM-SpMM);
 *                            C dense;   the product B*C is "the intermediate" T.
 *
 * All functions return 0 on success or a negative tf_status; the text of the last
 * error on the calling thread is available from tf_last_error_string().
 */
#ifndef TILEFUSION_HIP_H
#define TILEFUSION_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int tf_status;
enum {
  TF_OK = 0,
  TF_EINVAL = -1,       /* bad argument (null pointer, negative size, shape mismatch)      */
  TF_EHIP = -2,         /* a HIP runtime call failed (no device, launch failure, ...)       */
  TF_ENOMEM = -3,       /* host or device allocation failed                                 */
  TF_ESCHEDULE = -4,    /* schedule is invalid or does not belong to these operands         */
  TF_EUNSUPPORTED = -5  /* shape outside what the kernels take (e.g. N not a multiple of 4) */
};

/* The reference has no error channel (void executors, exit(1) in its drivers,
 * fusion/src/Fusion_Utils.cpp:208-211); this is the replacement. */
const char *tf_last_error_string(void);

/* Library version "major.minor". */
const char *tf_version(void);

/* ---- device ----------------------------------------------------------------- */

/* Structs the library fills in for the caller ("out-structs": tf_device_info, tf_schedule_info,
 * tf_schedule_view, tf_profile) start with struct_size, which the CALLER sets to sizeof(the struct)
 * as it was compiled before the call.  Fields are only ever appended, so the library writes the
 * first min(struct_size, its own sizeof) bytes and nothing behind them: a caller built against an
 * older header keeps working and its stack is not overrun.  TF_EINVAL when struct_size is smaller
 * than the struct's first version (stated at each struct) -- which includes a forgotten 0. */
typedef struct {
  size_t struct_size;      /* set by the caller; first version: through xcd_round_robin */
  int device;              /* HIP device ordinal in use                           */
  int compute_units;       /* 256 on MI355X                                       */
  int xcds;                /* accelerator complex dies sharing an L2 each (8)     */
  int lds_bytes_per_block; /* max LDS one workgroup may take (163840 on gfx950)   */
  int wavefront;           /* 64                                                  */
  int clock_khz;
  size_t hbm_bytes;
  char arch[64];           /* "gfx950..."                                         */
  int xcd_round_robin;     /* 1: a probe launch found workgroup b on the XCD of workgroup b mod xcds and
                              those xcds distinct -- what the kernels that pin work to an XCD's L2 rely on
                              (column-partitioned long rows, runs of neighbouring tiles); 0: it did not
                              (results stay right, that locality is lost); -1: the probe could not run  */
} tf_device_info;

/* Selects the device for the calling thread and reports its properties.  Optional:
 * every other entry point works on the current HIP device. */
tf_status tf_device_init(int device, tf_device_info *info);
tf_status tf_device_synchronize(void);

/* Measurement aid, no counterpart in the reference: one workgroup of eight wavefronts per compute unit, two per SIMD,
 * each running `iters` rounds of 32 v_mfma_f32_16x16x4_f32 (role 1), 256 v_fma_f32 (role 2), 32
 * v_mfma_f32_16x16x32_bf16 (role 3) or nothing (role 0); `role_older` is what the first four wavefronts (the older one
 * of every SIMD) do, `role_younger` the other four.  *ms = average duration of five launches.  Tells whether the
 * fp32 MFMA path and the VALU of a SIMD work at the same time (they do not: durations add), which bounds every kernel
 * that runs the GEMM beside the gathers.  Allocates and synchronizes: not for a timed path. */
tf_status tf_calibrate_issue(int role_older, int role_younger, int iters, float *ms);

/* Streams and events are passed as void* so that callers need no HIP headers; a
 * stream argument of NULL is the default stream.  A hipStream_t obtained elsewhere
 * (e.g. torch.cuda.current_stream().cuda_stream) can be passed as is. */
tf_status tf_stream_create(void **stream);
tf_status tf_stream_destroy(void *stream);
tf_status tf_stream_synchronize(void *stream);
tf_status tf_event_create(void **event);
tf_status tf_event_destroy(void *event);
tf_status tf_event_record(void *event, void *stream);
tf_status tf_event_synchronize(void *event);
tf_status tf_event_elapsed_ms(void *start, void *stop, float *ms);

/* ---- operands ---------------------------------------------------------------- */

/* Device-resident CSR matrix.  Stands in for sym_lib::CSR {m,n,nnz,p,i,x} as the
 * executors receive it (fusion/src/SpMM_SpMM_vectorized.cpp:876-880: Ap, Ai, Ax). */
typedef struct tf_csr tf_csr;
/* Device-resident dense row-major matrix (the reference's bare float* operands). */
typedef struct tf_dense tf_dense;

/* Copies a host CSR to the device.  Column indices need not be sorted. */
tf_status tf_csr_upload(int M, int N, const int *Ap, const int *Ai, const float *Ax,
                        tf_csr **out);
/* Wraps CSR arrays that already live in device memory; nothing is copied or owned. */
tf_status tf_csr_wrap_device(int M, int N, int nnz, const int *dAp, const int *dAi,
                             const float *dAx, tf_csr **out);
/* 64-bit fingerprint of a sparsity pattern (row pointers and column indices, host arrays); never 0.
 * tf_csr_upload and tf_inspect compute it, and the executors compare: a schedule is only run on
 * operands with the pattern it was built from (TF_ESCHEDULE otherwise).  The reference has no
 * such check: its executors trust whatever schedule they are handed. */
uint64_t tf_pattern_hash(int M, const int *Ap, const int *Ai);
/* A wrapped matrix has no host arrays to fingerprint, so its pattern is not checked unless the
 * caller, who knows the host copy, provides the fingerprint here (0 = unknown again). */
tf_status tf_csr_set_pattern_hash(tf_csr *a, uint64_t hash);
void tf_csr_free(tf_csr *a);

tf_status tf_dense_upload(int M, int N, const float *host, tf_dense **out);
tf_status tf_dense_alloc(int M, int N, tf_dense **out); /* contents undefined */
tf_status tf_dense_wrap_device(int M, int N, float *dptr, tf_dense **out);
tf_status tf_dense_download(const tf_dense *d, float *host);
tf_status tf_dense_fill(tf_dense *d, float value, void *stream);
/* dst = src (same shape), device to device on the given stream.  No counterpart in the reference
 * (its operands never leave host memory); used to keep results on the device and by the
 * benchmark's counter calibration. */
tf_status tf_dense_copy(tf_dense *dst, const tf_dense *src, void *stream);
float *tf_dense_device_ptr(const tf_dense *d);
void tf_dense_free(tf_dense *d);

/* ---- matrices from files -------------------------------------------------------- */

/* Reads a sparse matrix into host CSR arrays (sorted columns, duplicates summed) that the
 * caller releases with tf_host_free.  By file extension, as get_matrix_from_parameter does
 * (fusion/src/Fusion_Utils.cpp:254-272):
 *   .mtx   MatrixMarket coordinate or array, real / integer / pattern (pattern entries are 1);
 *          symmetric and skew-symmetric files are expanded to the full matrix, which the
 *          reference's drivers do with make_full before use (SpMM_SpMM_SP_Demo.cpp:24-32);
 *   .smtx  DLMC: "rows, cols, nnz", the row pointers, the column indices; every value is 1
 *          (readSparseMatrix, Fusion_Utils.cpp:205-250).
 * Host-only; no GPU is needed. */
tf_status tf_read_matrix(const char *path, int *M, int *N, int *nnz, int **Ap, int **Ai, float **Ax);
/* The same file kinds as a dense row-major matrix (the feature matrices of the GCN drivers,
 * read_mtx_array_real at Fusion_Utils.cpp:283). */
tf_status tf_read_dense(const char *path, int *M, int *N, float **data);
void tf_host_free(void *p);

/* ---- reordering ------------------------------------------------------------------ */

/* Reverse Cuthill-McKee ordering of a square matrix' pattern, symmetrised (A + A^T): rows
 * that depend on each other end up close together, so that tiles can fuse them.  The
 * reference reorders its inputs offline with scipy's reverse_cuthill_mckee
 * (fusion/scripts/reorder_graphs.py:3,21).  perm[new index] = old index, M entries.  Every
 * component starts from a pseudo-peripheral node; components are taken in order of their
 * smallest-degree node.  Host-only. */
tf_status tf_reorder_rcm(int M, const int *Ap, const int *Ai, int *perm);
/* Partition-based ordering of a square matrix' pattern, symmetrised: n_parts parts of (almost) equal size, each
 * grown breadth-first from a seed so that most edges stay inside a part, one after the other in perm; vertices
 * with more than hub_degree neighbours (0 = sixteen times the mean degree, at least 64) are set aside first and
 * placed in front, by falling degree -- on a power-law graph they would otherwise pull every part into one blob,
 * and in front they make the most-read intermediate rows one stretch of memory.  Stands in for the reference's
 * graph-partitioner ordering (METIS metis_perm_general, fusion/src/Fusion_Utils.cpp:181-203; the partitioner itself
 * is not part of the reference tree): greedy graph growing, its classical initial partitioner.
 * perm[new index] = old index, M entries.  part_ptr (may be null): n_parts + 2 entries, [0, part_ptr[1]) are the
 * hubs, part p is [part_ptr[p + 1], part_ptr[p + 2]).  Host-only. */
tf_status tf_reorder_partition(int M, const int *Ap, const int *Ai, int n_parts, int hub_degree, int *perm, int *part_ptr);
/* B = A[perm,:][:,perm] (reorder_graphs.py:22), columns sorted; the arrays are released with
 * tf_host_free.  With C' = C[perm,:], D' = B (B C') is D[perm,:] of D = A (A C). */
tf_status tf_permute_csr(int M, const int *Ap, const int *Ai, const float *Ax, const int *perm, int **Bp, int **Bi,
                         float **Bx);

/* ---- inspector ---------------------------------------------------------------- */

enum { TF_OP_SPMM_SPMM = 0, TF_OP_GEMM_SPMM = 1 };

/* Parameters of the gfx950 schedule.  Zero in any field (but struct_size) means "default". */
typedef struct {
  size_t struct_size;    /* sizeof(tf_inspect_opts) as the caller was compiled; fields are only
                            ever appended, so the library reads this many bytes and takes the
                            defaults for fields a caller built against an older header does not
                            have.  Must be set (TF_EINVAL when it is 0 or too small to hold N). */
  int op;                /* TF_OP_SPMM_SPMM or TF_OP_GEMM_SPMM                               */
  int N;                 /* columns of C and D (reference: bCols / EmbedDim).  Any N > 0.  The
                            MFMA kernels of GeMM-SpMM take 32, 64 .. 256 columns: for any other
                            N the schedule is built for equal column panels of such a width
                            (48 -> one of 64, 300 -> two of 160) and the executor runs one pass
                            per panel through a panel of C and of D in the schedule's workspace */
  int K;                 /* GeMM-SpMM: columns of dense B = rows of C (FeatureDim); else 0.
                            Any K > 0: the kernels step k by 8, so for other K the executor
                            copies B and C, zero-padded to the next multiple of 8, into the
                            schedule's workspace on every call (counted in workspace_bytes) */
  int lds_budget_bytes;  /* LDS one fused tile may take; plays the role of the cache budget
                            ScheduleParameters::TileM of the reference's variable-tile
                            inspector.  Default 65536 (81920 when an inner pattern is
                            given; GeMM-SpMM: 163840 when the streamed kernel applies, that
                            is K <= 256, N <= 128 or K <= 128, and a ring of 256 rows fits),
                            max 163840.                                                       */
  int tile_rows;         /* cap on the rows a tile owns; default: sized so that the launch
                            has about four tiles per compute unit                             */
  float max_redundancy;  /* a tile may compute up to this many intermediate rows per owned
                            row (halo rows recomputed so that boundary rows still fuse);
                            1.0 disables recomputation = the reference's tiling.
                            Default 3.0 for SpMM-SpMM, 1.5 for GeMM-SpMM.                    */
  int long_row_nnz;      /* remainder rows with more stored entries than this are worked on by a
                            whole workgroup each (in chunks of max(this, 1024) entries, partial
                            sums added in a fixed order); default 32 -- 64 where the long rows are
                            regrouped by column partition (long_row_partition) --, max 2048    */
  int compute_units;     /* sizing hint; default: the current device, or 256 with no device  */
  /* SpMM-SpMM only, optional: sparsity pattern of the inner matrix B (M x inner_cols, host
     arrays).  In every run of the reference B is A (fusion/example/SpMM_SpMM_Demo_Utils.h:
     53-54); pass A's arrays again for that case.  With it the inspector can tell when the rows
     of C a tile reads form a small contiguous window and then stages that window in LDS
     ("windowed" tiles: both products run out of LDS).  Null = unknown, C is gathered from HBM. */
  const int *inner_Ap;
  const int *inner_Ai;
  int inner_cols;
  int strip_cols;        /* windowed tiles work on this many columns of C/D at a time (32 or 64);
                            default 32                                                         */
  int xcd_chunk_rows;    /* how the row kernels' workgroups are dealt to the 8 XCDs: 0 = round-robin
                            (default), n > 0 = chunks of n rows per XCD turn (a 3D stencil with
                            plane distance d keeps its halo in one L2 with n = d/8), -1 = one
                            contiguous run of rows per XCD                                     */
  int wide_strips;       /* which kernel runs windowed tiles: 1 = strips of 64 columns (N % 64 == 0),
                            one workgroup of 1024 threads and up to 160 KB of LDS per tile, the
                            entries read from the CSR arrays in place (LDS rows of 256 bytes are
                            read without bank conflicts), tile_rows defaults to rows / compute
                            units; -1 = strips of strip_cols columns, the tile's entries staged in
                            LDS, two workgroups per compute unit; 0 = the first when N % 64 == 0 and
                            strip_cols, tile_rows and lds_budget_bytes are left at 0, else the
                            second                                                             */
  int long_row_partition; /* long remainder rows (more than long_row_nnz entries): 1 = regroup their entries
                            by column so that each XCD gathers from its own part of the most-read
                            intermediate rows, which then stays in its L2 (power-law graphs); -1 = cut
                            them into chunks of consecutive entries; 0 = the first when the long rows
                            hold a million entries or more and the intermediate exceeds 64 MB.
                            With 1 the schedule keeps A's values in the regrouped order (what the
                            reference's reordered adjacency, createReorderedAdj in
                            fusion/gcn/SingleLayer/GCN_Single_Layer_SP_Demo_Utils.h:618-653, is to its
                            executors): built on the first call with a matrix from tf_csr_upload, whose
                            device arrays never change, and on every call with one from
                            tf_csr_wrap_device, whose owner may change them between calls            */
  /* SpMM-SpMM with an inner pattern, N a multiple of 64, rows of at most 32 entries: marching runs for
     patterns whose dependences no range of consecutive rows holds (stencils on a 3D grid).  A run is a
     column of march_tile_x x march_tile_y grid points that one workgroup walks plane by plane, keeping
     the rows of C and of the intermediate that the coming planes need in LDS and recomputing the
     intermediate's halo ring -- tiling with redundancy as in the reference's
     fusion/src/SpMM_SpMM.cpp:984-1057, for rows that are not neighbours in memory.
     march: 0 = where windowed tiles do not apply and a grid is known, 1 = the same (tf_inspect fails if
     no marching schedule can be built), -1 = never.  grid_nx/ny/nz: the grid the rows are the points
     of, x fastest (their product must be the row count); all 0 = found from the pattern when it is a
     7-point-like stencil (row-to-column distances 1, nx, nx*ny).  The grid only deals rows to runs:
     what a run loads, recomputes and keeps is derived from the patterns and checked by
     tf_schedule_validate_inner, so a wrong grid cannot give wrong results.  march_tile_x/y: 0 = the
     largest column whose rows fit LDS (8 x 8 on a 7-point stencil). */
  int march;
  int grid_nx, grid_ny, grid_nz;
  int march_tile_x, march_tile_y;
  /* Remainder rows (second-op rows served from the intermediate in HBM) are worked on in the order of
     a list (by length class).  0 / 1 = when that order is not simply all rows in order, the schedule
     also keeps those rows' columns -- and the executor their values -- side by side in list order,
     which is what the reference's reordered adjacency is to its executors (createReorderedAdj,
     fusion/gcn/SingleLayer/GCN_Single_Layer_SP_Demo_Utils.h:618-653, read by
     forwardForOneLayerFusedParallelSeparatedReorderedAdjVectorizedSP, GCN_Layer_MKL_Forward_Utils.h:294-373);
     -1 = the rows are read from A's arrays in place through the list. */
  int reorder_adjacency;
  /* Column-partitioned long rows (long_row_partition): bytes of most-read intermediate rows dealt to each of
     the 8 XCD partitions; default 12 MB, three times an XCD's L2 (the reads inside a partition are skewed
     too, and its hottest rows are what stays). */
  int hot_partition_bytes;
  /* Short remainder rows kept in list order (reorder_adjacency) on a graph with hub rows: bytes of most-read
     intermediate rows that those rows' gathers may keep in an L2; gathers of all other rows are marked in the
     schedule and fetched with streaming loads, so that rows read once do not push out rows with readers.
     0 = 32 MB when the long rows are column-partitioned (long_row_partition: a power-law graph), else off;
     -1 = off; n > 0 = n bytes.  Only when N is a multiple of 4, and only if the set takes a quarter of the reads. */
  int short_row_hot_bytes;
  /* GeMM-SpMM schedules of a square matrix with K and N of 32, 64 or 128 also get two-layer tiles when the pattern
     allows (every tile's halo of hidden rows and the halo of those fit LDS: banded or reordered patterns): what
     tf_gcn_two_layers runs when the schedule serves as its second layer's.  0 = build them, -1 = do not. */
  int two_layer_tiles;
  /* GeMM-SpMM schedules in which nothing fuses (the step is a GEMM of the intermediate rows that are read, then
     gathers through the schedule's own lists): the intermediate's rows are stored in the order in which they are
     read most -- the rows of the hot partitions first, then by falling number of reads -- instead of at their own
     index.  Invisible to the caller (results identical); 0 = do so, -1 = rows at their own index. */
  int place_intermediate;
} tf_inspect_opts;

typedef struct tf_schedule tf_schedule;

/* Builds the fused-tile schedule for D = A*(B*C) from the sparsity pattern of A
 * (host arrays; A is L x M, the intermediate has M rows).  Pure host work: no GPU is
 * needed.  Replaces InspectorForTileFusedCSRVariableTileSize::
 * generateVariableTileSizeScheduleGeMMSpMM (fusion/include/sparse-fusion/
 * Fusion_Inspector.h:850-1017) and ...ForBothWavefronts (:676-846): same roles
 * (tiles own contiguous first-op rows; a second-op row is fused into a tile iff all
 * its column indices lie in the rows the tile computes; everything else goes to an
 * unfused remainder), re-derived for one workgroup's LDS instead of a CPU cache. */
tf_status tf_inspect(int L, int M, const int *Ap, const int *Ai, const tf_inspect_opts *opts,
                     tf_schedule **out);
void tf_schedule_free(tf_schedule *s);

typedef struct {
  size_t struct_size;    /* set by the caller; first version: through march_slots   */
  int op, N, K;
  int rows;              /* L: rows of A / D                                        */
  int inter_rows;        /* M: rows of the intermediate                             */
  int n_tiles;
  int n_fused_rows;      /* second-op rows served from LDS                          */
  int n_remainder_rows;  /* second-op rows served from the intermediate in HBM      */
  int n_long_rows;       /* of those, rows split into chunks                        */
  int n_long_chunks;     /* chunks of consecutive entries, or column-partitioned segments */
  int n_producer_rows;   /* sum over tiles of rows computed (>= M with recomputation) */
  int n_writeback_rows;  /* intermediate rows that are written to HBM               */
  int max_tile_producer_rows;
  int lds_bytes;         /* dynamic LDS of the fused-tile kernel                    */
  int windowed;          /* 1 when tiles stage their window of C in LDS             */
  int strip_cols;        /* columns per strip of the windowed kernel, else 0        */
  int xcd_chunk_rows;    /* rows per XCD turn of the row kernels (0: round-robin, -1: contiguous) */
  int streamed;          /* 1 when GeMM-SpMM tiles are long runs streamed through an LDS ring */
  int ring_rows;         /* intermediate rows the ring holds, else 0                 */
  int wide_strips;       /* 1 when windowed tiles run on the 64-column, 1024-thread kernel */
  int long_row_hot_cols; /* intermediate rows kept in the XCDs' L2 partitions for the long rows, else 0 */
  long long fused_nnz;   /* stored entries of A in fused rows (getFusedNnzNum)      */
  long long workspace_bytes; /* device memory the executor keeps (intermediate + partials) */
  int marched;           /* 1 when the tiles are marching runs                       */
  int march_tile_x, march_tile_y; /* grid points of a run per plane                    */
  int march_slots;       /* LDS slots (64-column rows) the fullest run uses          */
  /* appended after the first version */
  int march_declined;    /* TF_MARCH_*: whether marching runs were built, and if not, why */
  int register_weights;  /* 1 when GeMM-SpMM tiles keep C in registers (fused_gemm_spmm_regw_kernel) */
  int n_zero_rows;       /* second-op rows without entries that a fill kernel clears (counted in n_remainder_rows) */
  int two_layer_tiles;   /* GeMM-SpMM: tiles that can carry their rows through two layers (tf_gcn_two_layers), else 0 */
  int short_row_hot_rows; /* intermediate rows whose gathers by the short remainder rows are left cacheable
                            (short_row_hot_bytes), else 0                                                    */
  int n_computed_rows;   /* intermediate rows the executor computes per call: the producer rows of the tiles it
                            launches (halo rows included) plus, for tiles that fuse nothing, only the rows some
                            remainder row reads -- on a graph with isolated nodes fewer than inter_rows       */
  int intermediate_placed; /* 1 when the intermediate's rows are stored in the order they are read most (place_intermediate) */
} tf_schedule_info;

/* tf_schedule_info.march_declined */
enum {
  TF_MARCH_BUILT = 0,         /* the schedule's tiles are marching runs                                     */
  TF_MARCH_NOT_TRIED = 1,     /* not SpMM-SpMM with an inner pattern, march = -1, or windowed tiles applied */
  TF_MARCH_SHAPE = 2,         /* A or B not square with the same row count, or N not a multiple of 64       */
  TF_MARCH_ROW_TOO_LONG = 3,  /* a row of A or B has more than 32 entries                                  */
  TF_MARCH_NO_GRID = 4,       /* grid_nx/ny/nz do not multiply to the row count, or none given and the
                                 pattern is not a 5- or 7-point-like stencil a grid can be read off      */
  TF_MARCH_NO_FIT = 5         /* no column of grid points whose rows fit LDS and the run tables            */
};

tf_status tf_schedule_get_info(const tf_schedule *s, tf_schedule_info *info);

/* The schedule in the layout of sym_lib::MultiDimensionalSet
 * (fusion/include/sparse-fusion/MultiDimensionalSet.h:15-21, as filled at
 * Fusion_Inspector.h:959-1010): n1 = 2 levels; level 0 = fused tiles, level 1 =
 * remainder partitions of up to 64 rows (one wavefront's row group);
 * ptr1[3], ptr2[P+1], ker_begin[2P], id[n_id], type[n_id].  First-op ids of a tile are
 * the rows it OWNS (each intermediate row is owned by exactly one tile); recomputed
 * halo rows are not listed there but are given by tile_range.
 * tile_range[4*t + {0,1,2,3}] = producer_begin, producer_end, own_begin, own_end.
 * Pointers are views into the schedule, valid until tf_schedule_free. */
typedef struct {
  size_t struct_size;   /* set by the caller; first version: through n_step_ptr */
  int n1, n_part, n_id, n_tiles;
  const int *ptr1, *ptr2, *ker_begin, *id, *type;
  const int *tile_range;
  const int *writeback; /* [2*n_tiles] begin,end of intermediate rows a tile stores to HBM */
  /* Streamed GeMM-SpMM schedules only (else null / 0): a tile is a long run produced 64 rows
     a step; tile_step[t] = first entry of tile t in step_ptr, or -1 if it fuses nothing.  With
     steps = ceil((producer_end - producer_begin) / 64), the fused rows computed while step q
     is produced are fused ids [step_ptr[tile_step[t] + q], step_ptr[tile_step[t] + q + 1])
     of the tile, q = 0..steps (step `steps` comes after the last production step); offsets
     count from the tile's first fused id, i.e. from id[ker_begin[2t]]. */
  const int *tile_step;
  const int *step_ptr;
  int n_step_ptr;
  /* appended after the first version */
  /* Two-layer tiles (tf_schedule_info.two_layer_tiles of them, else null / 0): two_layer_range[8*t + {0..5}] =
     o0, o1, h0, h1, t0, t1: tile t owns the rows [o0, o1) of D, computes the hidden rows [h0, h1) they read and
     the rows [t0, t1) of the first layer's intermediate those read ([8*t + 6], [8*t + 7]: where its second slab and its copy of A's
     rows start in LDS, in floats). */
  const int *two_layer_range;
  int n_two_layer;
} tf_schedule_view;

tf_status tf_schedule_get_view(const tf_schedule *s, tf_schedule_view *view);

/* Exact check of a schedule against the pattern it was built from: every first-op
 * row owned once, every second-op row scheduled once, every fused row's columns
 * inside its tile's producer range, every remainder row's columns covered by a
 * write-back range, LDS budget respected.  Returns TF_ESCHEDULE with a message
 * naming the first violation.  (The reference never checks its schedules.) */
tf_status tf_schedule_validate(const tf_schedule *s, int L, int M, const int *Ap,
                               const int *Ai);
/* The same, and for a schedule built with an inner pattern (tf_inspect_opts.inner_Ap) also
 * what only that pattern shows: every windowed tile's window of C holds all rows its producer
 * rows read, and window, slab and tables fit the LDS the kernel is launched with. */
tf_status tf_schedule_validate_inner(const tf_schedule *s, int L, int M, const int *Ap, const int *Ai,
                                     const int *inner_Ap, const int *inner_Ai, int inner_cols);

/* ---- executors ---------------------------------------------------------------- */

enum {
  TF_ACCUMULATE = 1u,   /* D += A*(B*C), the reference's convention (its callers zero D
                           first); without it D is overwritten and need not be initialised */
  TF_SECOND_STREAM = 2u, /* GeMM-SpMM with column-partitioned long rows: run the hot long-row segments
                           on a second stream of the schedule's own (same priority), forked from and
                           joined to the given one with events, beside the GEMM of the other rows.
                           Without it every kernel of a call runs on the given stream, one after
                           another -- which measured as fast on the R-MAT configuration (2.32 ms
                           against 2.35 ms: the gathers and the GEMM's operand traffic meet in the
                           same memory system), so it is not the default */
  TF_RELU = 4u,          /* tf_gcn_two_layers: ReLU between the layers */
  TF_FUSE_LAYERS = 8u    /* tf_gcn_two_layers: run the second schedule's two-layer tiles (one launch, the hidden
                           layer never leaves LDS), or fail with TF_EUNSUPPORTED if it has none; without this flag
                           each layer is one tf_gemm_spmm (see tf_gcn_two_layers)                            */
};

/* D = A * (B * C), A and B sparse.  Stands in for
 * swiftware::sparse::spmmCsrSpmmCsrFusedVectorized2_32SP
 * (fusion/src/SpMM_SpMM_vectorized.cpp:876-989; the reference names the inner
 * matrix "A" and the outer one "B", the README and this ABI name them the other way
 * round).  A is L x M, B is M x Kc, C is Kc x N, D is L x N.  The schedule must come
 * from tf_inspect on A's pattern with op = TF_OP_SPMM_SPMM and the same N.
 * Asynchronous on `stream`.  One call at a time per schedule (it owns the workspace). */
tf_status tf_spmm_spmm(const tf_csr *A, const tf_csr *B, const tf_dense *C, tf_dense *D,
                       tf_schedule *schedule, unsigned flags, void *stream);

/* D = A * (B * C), A sparse, B and C dense.  Stands in for
 * forwardForOneLayerFusedParallelSeparatedVectorizedSP
 * (fusion/gcn/GCN_Layer_MKL_Forward_Utils.h:218-291): B is M x K (Features), C is
 * K x N (Weight, not transposed), D is L x N.  The tile GEMM runs on fp32 MFMA. */
tf_status tf_gemm_spmm(const tf_csr *A, const tf_dense *B, const tf_dense *C, tf_dense *D,
                       tf_schedule *schedule, unsigned flags, void *stream);

/* Two GCN layers in one call:  D = A * (act(A * (X * W1)) * W2),  act = ReLU with TF_RELU, else
 * the identity.  Stands in for fusedGCN (binding-project/src/Functions.cpp:228-290) and for what the
 * reference's end-to-end model runs (binding-project/gcn-e2e-training/FusedGCNModule.py:7-18: two fused
 * layers with a ReLU between).  A is square (M x M), X is M x K, W1 is K x H, W2 is H x N (weights not
 * transposed, as in tf_gemm_spmm), D is M x N.  s1 must come from tf_inspect on A's pattern for
 * (TF_OP_GEMM_SPMM, K, H), s2 for (TF_OP_GEMM_SPMM, H, N); they may be one schedule when K = H = N.
 * The hidden layer stays on the device.  Two ways to run, chosen per call:
 *  - two-layer tiles (fused_gcn2_kernel; the reference's "four kernels per tile", MixPtr[4j .. 4j+3] at Functions.cpp:
 *    228-290): when s2 carries them (tf_schedule_info.two_layer_tiles > 0: a square matrix whose rows' halos fit LDS
 *    -- banded or reordered patterns -- and H, N of 32, 64 or 128), K is a multiple of 8 up to 256 and `hidden` is
 *    null, ONE launch takes every tile through GEMM, SpMM, activation, GEMM, SpMM with the first intermediate, the
 *    hidden rows and the second intermediate in LDS; only X, the weights, A and D cross HBM.  Taken with
 *    TF_FUSE_LAYERS only: a tile recomputes the halo rows of its neighbours in both GEMMs (1.4x the GEMM rows on a
 *    band of 32 at H = N = 128) and runs its phases one after the other, which measured slower than the composed path
 *    wherever that one streams (0.63 ms against 0.31 ms on 262,144 rows, K = H = N = 128); what it saves is the hidden
 *    layer's trip through HBM (WRITE_SIZE = D only) and a launch;
 *  - composed (the default): each layer runs as tf_gemm_spmm does with its own schedule (rows fuse inside a layer), the hidden
 *    layer in `hidden` (M x H) when given -- training keeps it for the backward pass -- else in a buffer that s2
 *    owns, one small ReLU launch between the layers.
 * The reference's fusedGCN reads its second GEMM's input
 * from the first GEMM's output instead of from the first layer's (imRes1 at :262) and has no activation;
 * this entry point computes the composition its callers mean. */
tf_status tf_gcn_two_layers(const tf_csr *A, const tf_dense *X, const tf_dense *W1, const tf_dense *W2, tf_dense *D,
                            tf_schedule *s1, tf_schedule *s2, tf_dense *hidden, unsigned flags, void *stream);

/* Unfused building blocks, the reference's in-process baselines:
 * Y = A * X   (swiftware::sparse::spmmCsrParallel<float>, fusion/src/SpMM_SpMM.cpp:37-55) */
tf_status tf_spmm(const tf_csr *A, const tf_dense *X, tf_dense *Y, unsigned flags, void *stream);
/* Y = X * W   (the cblas_sgemm call at fusion/gcn/GCN_Layer_MKL_Forward_Utils.h:1144).
 * K % 8 == 0, N % 32 == 0 and N <= 256 go straight to the MFMA kernel; any other shape is padded / cut into column
 * panels in a workspace the library keeps per device.  The workspace only grows: a call whose buffers fit is
 * asynchronous on `stream` like every other; the first call with a larger shape frees and allocates (which waits for
 * the device, and is refused with TF_EUNSUPPORTED while `stream` is being captured).  Calls with such shapes on one
 * device share that workspace: keep them on one stream, or order them with events. */
tf_status tf_gemm(const tf_dense *X, const tf_dense *W, tf_dense *Y, void *stream);

/* D = A * (B * C), A and B sparse, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  It needs no schedule and calls no hipMalloc / hipFree: the two products run as two
 * row-kernel passes and the intermediate (B->M x C->N floats) lives in one fixed array of
 * tf_noalloc_scratch_bytes() bytes (32 MiB) that every GPU the library is loaded on holds until the
 * process ends; a larger intermediate is rejected with TF_EUNSUPPORTED.  All calls on one GPU
 * share that array: calls that overlap in time on one GPU (two streams, two threads) race and
 * give wrong results -- serialise them.  Nothing of an earlier call's contents is read.  Results
 * equal the reference's fma order exactly (rows of any length are walked in CSR order). */
tf_status tf_spmm_spmm_noalloc(const tf_csr *A, const tf_csr *B, const tf_dense *C, tf_dense *D,
                               unsigned flags, void *stream);
size_t tf_noalloc_scratch_bytes(void);

/* Benchmark aid, no counterpart in the reference (its harness times whole executor calls):
 * when switched on, the executors record events around every kernel launch of a call with this
 * schedule; tf_schedule_get_profile waits for the last call and reports each launch's name and
 * duration in ms (kernels that ran side by side on two streams each report their own). */
#define TF_PROFILE_MAX 16
typedef struct {
  size_t struct_size;   /* set by the caller; first version: through ms */
  int n;
  const char *name[TF_PROFILE_MAX];
  float ms[TF_PROFILE_MAX];
} tf_profile;
tf_status tf_schedule_set_profiling(tf_schedule *s, int enable);
tf_status tf_schedule_get_profile(tf_schedule *s, tf_profile *out);

#ifdef __cplusplus
}
#endif
#endif /* TILEFUSION_HIP_H */
