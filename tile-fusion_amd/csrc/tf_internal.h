// Internal declarations shared by the host-side inspector, the C ABI and the HIP
// kernels of libtilefusion_hip.  Not installed; the public surface is
// include/tilefusion_hip.h.
#pragma once
#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include "tilefusion_hip.h"

namespace tf {

// One fused tile = one workgroup.  The workgroup computes intermediate rows
// [prod_begin, prod_end) into LDS, stores rows [wb_begin, wb_end) of them to the
// intermediate in HBM (the ones remainder rows will read), then computes the
// second-op rows ids[cons_begin .. cons_end) out of LDS.
struct TileDesc {
  int prod_begin, prod_end;
  int own_begin, own_end;
  int wb_begin, wb_end;
  int cons_begin, cons_end;
};
static_assert(sizeof(TileDesc) == 32, "TileDesc is read as two int4 by the kernels");

// A chunk of one long remainder row: stored entries [k_begin, k_end) of `row`,
// reduced by a whole workgroup into partial[slot].
struct LongChunk {
  int row, k_begin, k_end, slot;
};
// All partials of one long row: D[row] = sum partial[first .. first+count).
struct LongRow {
  int row, first, count, pad;
};

// A tile that carries its rows through two GCN layers (tf_gcn_two_layers): it owns the rows [o0, o1) of D, which
// read the rows [h0, h1) of the hidden layer, which read the rows [t0, t1) of the first layer's intermediate.
struct Tile2 {
  int o0, o1, h0, h1, t0, t1;
  int b_off;  // floats of LDS in front of the tile's slab B (its slab A: the first intermediate, then the second)
  int c_off;  // ... and in front of its copy of A's rows [min(o0, h0), max(o1, h1)): row pointers, columns, values
};
static_assert(sizeof(Tile2) == 32, "Tile2 is read as two int4 by the kernel");
constexpr int kTile2Pad = 4;                 // floats behind every slab row (tf_gcn2.hip: kG2Pad)
constexpr int kTile2StageFloats = 2 * 64 * 36;  // the two staging buffers of X (tf_gcn2.hip: kG2StageFloats)

struct DeviceSchedule;  // device copies + workspace, defined in tf_api.cpp

// Marching runs: LDS layout and list format shared by the inspector, the validator and the kernel.
constexpr int kMarchW = 8;               // entries per ELL row when no row of either pattern has more: a lane of a quad holds two
constexpr int kMarchWideW = 32;          // ... and when one has (up to 32: longer rows do not march): a lane of a group holds two
// entries per ELL row in a schedule whose longest row has `width` entries
constexpr int march_ell_stride(int width) { return width <= kMarchW ? kMarchW : kMarchWideW; }
constexpr int kMarchRowBytes = 256;      // an LDS slot: 64 columns of one row
constexpr int kMarchTabBytes = 4096;     // per-iteration table of a run, staged at the start of LDS
constexpr int kMarchMaxIter = kMarchTabBytes / 16 - 2;  // (16 bytes of table per iteration)
constexpr int kMarchZeroOff = kMarchTabBytes;                    // a row of zeros, read by padding entries
constexpr int kMarchTrashOff = kMarchTabBytes + kMarchRowBytes;  // a row that takes what lane groups without work write
constexpr int kMarchSlot0 = kMarchTabBytes + 2 * kMarchRowBytes; // first slot
constexpr int kMarchSrcA = 1 << 30;      // flag in march_ell_src: the value is one of A's (else of B's)
constexpr int kMarchGroups = 32;         // lane groups (of 16 lanes) per workgroup
// rows one lane group takes per iteration, at most (the kernel's register sets): intermediate rows,
// second-op rows, rows of C
constexpr int kMarchTpg = 3, kMarchDpg = 2, kMarchLpg = 5;

}  // namespace tf

struct tf_schedule {
  tf_inspect_opts opts{};  // resolved (no zero "default" fields left)
  int L = 0, M = 0;
  int lds_bytes = 0;          // dynamic LDS of the fused kernel: intermediate slab (+ GEMM staging)
  int lds_bytes_general = 0;  // the same for the kernel that gathers C from HBM (fallback of windowed tiles)
  bool windowed = false;      // tiles stage their window of C in LDS (win holds the windows)
  bool win_wide = false;      // ... in 64-column strips on the 1024-thread kernel (entries read in place)
  long long inner_nnz = 0;    // stored entries of the inner pattern the windows were built from
  std::vector<int> win;       // [2*n_tiles] first,last+1 row of C read by the tile's producer rows
  int slab_rows = 0;          // max producer rows of any tile
  int user_K = 0;             // K as given; opts.K is K rounded up to a multiple of 8 (what the kernels see)
  int user_N = 0;             // N as given; GeMM-SpMM with a width the MFMA kernels do not take (N % 32, N > 256) runs
  int n_panels = 1;           // as n_panels column panels of opts.N columns each, the last one zero-padded
  int gemm_kc = 0;            // rows of C staged in LDS per step (GeMM-SpMM)
  bool gemm_regw = false;     // GeMM-SpMM tiles keep C in registers (no staging; slab rows padded)
  int slab_ld = 0;            // floats between two slab rows of the general / GeMM-SpMM tile kernels
  bool gemm_stream = false;   // GeMM-SpMM tiles are long runs streamed through a ring of ring_rows slab rows
  int ring_rows = 0;
  int stream_step_cap = 0;    // rows a step of a streamed run may hold (all but the last step)
  int stream_max_len = 0;     // entries a fused row of a streamed run may have
  std::vector<int> tile_step;    // per tile: first entry of its steps in step_ptr (-1: fuses nothing)
  std::vector<int> launch_step;  // the same for launch_tiles
  std::vector<int> step_ptr;     // per streamed tile steps+2 offsets into fused_ids: rows of step q are
                                 // [step_ptr[q], step_ptr[q+1]), computed while rows 64q.. are produced
  std::vector<int> view_step_ptr;  // step_ptr with offsets counted from each tile's first fused id
  std::vector<int> fused_rec;    // (row, first entry, end, 0) per fused id of a streamed schedule
  std::vector<tf::TileDesc> tiles;
  std::vector<tf::TileDesc> launch_tiles;  // the tiles that fuse something: one workgroup each
  std::vector<int> plain_rows;      // intermediate rows of tiles that fuse nothing, computed by the
                                    // row kernels -- only the rows some remainder row reads
  int plain_hot = 0;                // with long_part: the first plain_hot of them are the rows of the hot
                                    // partitions (produced first, so that the hot segments can start early)
  bool profiling = false;           // executors record events around every launch
  std::vector<int> fused_ids;       // second-op rows per tile, tile after tile
  std::vector<int> rem_rows;        // remainder rows handled one row per lane group, ordered by
                                    // length class so that a workgroup's rows cost about the same
  bool rem_identity = false;        // rem_rows is 0..L-1 in order
  std::vector<int> zero_rows;       // second-op rows without entries, when many: their rows of D are cleared by a
                                    // fill kernel instead of taking a lane group each in the row kernel
  // When the list is not the identity, its rows are also kept as a CSR of their own in list order
  // (row q of it is row rem_rows[q] of A): rem_ptr [n + 1], rem_col, and rem_src = where each entry
  // sits in A's arrays (the executor copies the values from there).
  std::vector<int> rem_ptr, rem_col, rem_src;
  bool rem_flagged = false;  // rem_col carries the "cold" mark in the top bit of some columns (short_row_hot_bytes)
  int rem_hot_rows = 0;      // intermediate rows left unmarked
  int xcd_chunk_rows = 0;           // rows per XCD turn of the row kernels (0: one contiguous run per XCD)
  std::vector<tf::LongChunk> long_chunks;
  std::vector<tf::LongRow> long_rows;
  // Long rows cut by column instead (long_part): the most-read intermediate rows are dealt to 8
  // partitions, one per XCD, small enough to stay in that XCD's L2; a long row's entries are
  // regrouped into segments of one partition (or of none: "cold") and of at most 64 entries,
  // each worked on like a short row by the XCD that caches its partition.  long_rows then holds
  // first/count into lrow_seg.
  bool long_part = false;
  int seg_per_xcd = 0;            // hot segments per partition, padded with empty ones
  int hot_cols = 0;               // intermediate rows in the 8 partitions together
  std::vector<int> seg_ptr;       // [n_seg + 1] into seg_src/seg_col: partition 0's segments, 1's, ..., 7's, the cold ones
  std::vector<int> seg_src;       // per regrouped entry: its index in A's arrays
  std::vector<int> ent_src, ent_pos;  // the same pairs (index in A's arrays, regrouped position) sorted by the former
  std::vector<int> seg_col;       // per regrouped entry: its column
  std::vector<int> lrow_seg;      // per long row (first, count of tf::LongRow): the partial-sum slots it adds up, in order:
                                  // segments, or for a row of more than 32 segments groups of up to 32 of them
  std::vector<tf::LongRow> seg_groups;  // such groups: row = the group's slot (n_seg + its index), first/count into lrow_seg
  // Marching runs (SpMM-SpMM on stencil-like patterns whose dependences no contiguous tile holds): a run
  // is one workgroup that walks a sequence of steps (a column of grid points, plane by plane) and keeps
  // the rows of C and of the intermediate that its next rows need in numbered LDS slots of one
  // 64-column row each.  Iteration i of a run has the C rows of load list i in LDS, computes the ELL rows
  // [row_ptr[2i], row_ptr[2i+1]) -- the intermediate rows first needed by the run's step i, into slots
  // (halo rows of neighbouring runs are recomputed) -- and, after a barrier, the ELL rows
  // [row_ptr[2i+1], row_ptr[2i+2]) -- the second-op rows of step i, to D -- while the C rows of list i+1
  // go to their slots.  Every entry of an ELL row names the LDS byte offset of the row it reads; the
  // inspector assigns the slots so that a row stays until its last reader has run.
  bool march = false;
  // GeMM-SpMM schedules in which nothing fuses and every gather goes through the schedule's own copies of the columns:
  // t_pos[c] = where row c of the intermediate is stored (its place in plain_rows: the rows of the hot partitions
  // first, the others by falling number of reads), -1 for rows nobody reads.  Empty: rows at their own index.
  std::vector<int> t_pos;
  int march_declined = TF_MARCH_NOT_TRIED;  // why there are no marching runs (TF_MARCH_*), TF_MARCH_BUILT when there are
  int march_grid[3] = {0, 0, 0};     // the grid the runs were cut from (x fastest)
  int march_tile[2] = {0, 0};        // grid points per run and plane: x, y
  int march_slots = 0;               // LDS slots in use by the fullest run
  int march_width = tf::kMarchW;         // entries of the longest row of either pattern (the kernel takes only that many pairs of a row, five at least)
  int march_tpg = 0, march_dpg = 0, march_lpg = 0;  // intermediate rows / second-op rows / C rows a lane group handles per iteration, at most
  std::vector<int> march_runs;       // (first iteration, iterations) per run
  std::vector<int> march_row_ptr;    // [2 * iterations + 1] into the ELL rows
  std::vector<int> march_load_ptr;   // [iterations + 1] into the load list
  std::vector<int> march_load;       // (row of C, LDS byte offset) pairs
  std::vector<int> march_row_out;    // per ELL row: >= 0 row of D, < 0 ~(LDS byte offset) of an intermediate row
  std::vector<int> march_row_id;     // per ELL row: the matrix row it computes (of B when out < 0, of A otherwise)
  std::vector<int> march_ell_off;    // [march_ell_stride(march_width) per ELL row] LDS byte offset of the row read (the zero row for padding)
  std::vector<int> march_ell_src;    // ... and where its value comes from: index into B's values, or into A's
                                     // with kMarchSrcA set; -1 for padding (value 0)
  // Two-layer tiles (GeMM-SpMM schedules of a square matrix with K and N of 32, 64 or 128, when every tile's two
  // halos fit LDS): what tf_gcn_two_layers runs when this is the second layer's schedule.  l2_lds_bytes: the LDS
  // of the fullest tile (slab A in front, slab B -- X staging, then the hidden rows -- behind it).
  std::vector<tf::Tile2> l2_tiles;
  int l2_lds_bytes = 0;
  long long fused_nnz = 0;
  int n_writeback_rows = 0;
  long long n_producer_rows = 0;
  // MultiDimensionalSet-layout view
  std::vector<int> ptr1, ptr2, ker_begin, id, type, tile_range, writeback;
  // pattern fingerprint, checked by the executors against their operands
  long long nnz = 0;
  uint64_t pattern_hash = 0;  // tf_pattern_hash of the pattern the schedule was built from
  uint64_t inner_hash = 0;    // ... and of the inner pattern, when one was given (0: none)
  tf::DeviceSchedule *dev = nullptr;
};

namespace tf {

tf_status fail(tf_status code, const char *fmt, ...);

// Out-structs (tf_device_info, tf_schedule_info, tf_schedule_view, tf_profile) begin with the size the
// caller was compiled with.  `full` is the struct as this library knows it; the caller gets its first
// min(struct_size, sizeof(T)) bytes and keeps its own struct_size, so nothing is written behind a
// struct that is shorter than this library's.  min_size = the struct's size in its first version.
template <class T> tf_status emit_out(const char *who, T *out, T &full, size_t min_size) {
  const size_t have = out->struct_size;
  if (have < min_size)
    return fail(TF_EINVAL, "%s: struct_size is %zu, the struct's first version has %zu bytes (set struct_size to sizeof of the struct before the call)",
                who, have, min_size);
  full.struct_size = have;
  std::memcpy(static_cast<void *>(out), &full, have < sizeof(T) ? have : sizeof(T));
  return TF_OK;
}
// size of struct T up to and including its member m
#define TF_SIZE_THROUGH(T, m) (offsetof(T, m) + sizeof(((T *)nullptr)->m))
// tf_march.cpp: builds marching runs into S (returns false, S untouched, when the pattern does not
// suit them), and checks such a schedule exactly against both patterns.
bool build_march(tf_schedule *S, int M, const int *Ap, const int *Ai, const int *Bp, const int *Bi,
                 const tf_inspect_opts &o, const tf_inspect_opts &given);
tf_status validate_march(const tf_schedule *s, int M, const int *Ap, const int *Ai, const int *Bp, const int *Bi);
void release_device_schedule(DeviceSchedule *d);
int default_compute_units();

}  // namespace tf
