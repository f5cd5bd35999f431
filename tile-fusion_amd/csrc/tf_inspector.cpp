// Host-side inspector of libtilefusion_hip: builds the gfx950 fused-tile schedule
// from the sparsity pattern of A, and checks schedules exactly.
//
// Roles follow the reference's variable-tile inspector
// (fusion/include/sparse-fusion/Fusion_Inspector.h:850-1017 and :676-846): tiles own
// contiguous first-op rows, a second-op row is fused into its tile iff every column
// it reads is produced inside the tile, the rest is an unfused remainder.  What is
// different is the machine model: a tile is one workgroup whose intermediate slab
// must fit an LDS budget, tiles may recompute a few halo rows of the intermediate
// so that boundary rows still fuse, and the remainder is cut into wavefront-sized
// row groups plus chunks of very long rows.
#include <algorithm>
#include <numeric>
#include <climits>
#include <cstdio>
#include <cstddef>
#include <cstdlib>
#include <cstring>

#include "tf_internal.h"

namespace {

constexpr int kMaxLds = 163840;  // LDS per workgroup on gfx950

int ceil_div(int a, int b) { return (a + b - 1) / b; }


// Two-layer tiles for tf_gcn_two_layers (see tf_internal.h: Tile2, and tf_gcn2.hip).  Greedy: a tile's owned
// range grows row by row while the two slabs its halos need fit `budget_floats` of LDS.  H = the hidden width
// (this schedule's K), N its output width.  Leaves S->l2_tiles empty when some single row's halos do not fit
// (a pattern without a band: the composed path serves it).
void build_two_layer_tiles(tf_schedule *S, int M, const int *Ap, const int *Ai, int H, int N, int compute_units) {
  const long long budget_floats = kMaxLds / 4;
  std::vector<int> lo(M), hi(M);  // column extent per row: [lo, hi), empty rows lo = INT_MAX, hi = -1
  for (int i = 0; i < M; ++i) {
    int a = INT_MAX, b = -1;
    for (int k = Ap[i]; k < Ap[i + 1]; ++k) { a = std::min(a, Ai[k]); b = std::max(b, Ai[k] + 1); }
    lo[i] = a; hi[i] = b;
  }
  const int cap = std::max(32, ceil_div(M, std::max(1, compute_units)));
  std::vector<tf::Tile2> tiles;
  long long max_floats = 0;
  auto align4 = [](long long x) { return (x + 3) / 4 * 4; };
  for (int o0 = 0; o0 < M;) {
    int h0 = INT_MAX, h1 = -1, t0 = INT_MAX, t1 = -1, o1 = o0;
    long long fa = 0, fb = tf::kTile2StageFloats, fc = 0;
    while (o1 < M && o1 - o0 < cap) {
      const int nh0 = std::min(h0, lo[o1]), nh1 = std::max(h1, hi[o1]);
      int nt0 = t0, nt1 = t1;
      if (nh1 > nh0) {  // hidden rows that the new row adds on either side
        const int left_end = h1 > h0 ? h0 : nh1;
        for (int j = nh0; j < left_end; ++j) { nt0 = std::min(nt0, lo[j]); nt1 = std::max(nt1, hi[j]); }
        if (h1 > h0)
          for (int j = h1; j < nh1; ++j) { nt0 = std::min(nt0, lo[j]); nt1 = std::max(nt1, hi[j]); }
      }
      const long long PH = std::max(0, nh1 - nh0), P1 = std::max(0, nt1 - nt0);
      const long long a = std::max(P1 * (H + tf::kTile2Pad), PH * (N + tf::kTile2Pad));
      const long long b = std::max<long long>(PH * (H + tf::kTile2Pad), tf::kTile2StageFloats);
      // the tile's copy of A's rows: those it owns and the hidden rows, one stretch of the CSR arrays
      const int c0 = PH > 0 ? std::min(o0, nh0) : o0, c1 = PH > 0 ? std::max(o1 + 1, nh1) : o1 + 1;
      const long long c = align4(c1 - c0 + 1) + 2 * align4(Ap[c1] - Ap[c0]);
      if (a + b + c > budget_floats) break;
      h0 = nh0; h1 = nh1; t0 = nt0; t1 = nt1; fa = a; fb = b; fc = c;
      ++o1;
    }
    if (o1 == o0) return;  // one row alone does not fit
    tf::Tile2 t{};
    t.o0 = o0; t.o1 = o1;
    t.h0 = h1 > h0 ? h0 : 0; t.h1 = h1 > h0 ? h1 : 0;
    t.t0 = t1 > t0 ? t0 : 0; t.t1 = t1 > t0 ? t1 : 0;
    t.b_off = (int)fa;
    t.c_off = (int)(fa + fb);
    tiles.push_back(t);
    max_floats = std::max(max_floats, fa + fb + fc);
    o0 = o1;
  }
  S->l2_tiles.swap(tiles);
  S->l2_lds_bytes = (int)(max_floats * 4);
}

}  // namespace

// Multiply-xorshift over the row pointers and column indices; 0 is kept for "unknown".
extern "C" uint64_t tf_pattern_hash(int M, const int *Ap, const int *Ai) {
  if (M <= 0 || !Ap) return 0;
  uint64_t h = 0x9E3779B97F4A7C15ull ^ (uint64_t)(uint32_t)M;
  auto mix = [&h](const int *p, long long n) {
    for (long long k = 0; k < n; ++k) {
      h = (h ^ (uint32_t)p[k]) * 0xD6E8FEB86659FD93ull;
      h ^= h >> 32;
    }
  };
  mix(Ap, (long long)M + 1);
  if (Ai && Ap[M] > 0) mix(Ai, Ap[M]);
  return h ? h : 1;
}

extern "C" tf_status tf_inspect(int L, int M, const int *Ap, const int *Ai,
                                const tf_inspect_opts *user, tf_schedule **out) {
  if (!out) return tf::fail(TF_EINVAL, "tf_inspect: out is null");
  *out = nullptr;
  if (L <= 0 || M <= 0 || !Ap || !user) return tf::fail(TF_EINVAL, "tf_inspect: bad L/M/Ap/opts");
  if (Ap[0] != 0) return tf::fail(TF_EINVAL, "tf_inspect: Ap[0] != 0");
  for (int i = 0; i < L; ++i)
    if (Ap[i + 1] < Ap[i]) return tf::fail(TF_EINVAL, "tf_inspect: Ap not monotone at row %d", i);
  const long long nnz = Ap[L];
  if (nnz > 0 && !Ai) return tf::fail(TF_EINVAL, "tf_inspect: Ai is null");

  // Only the bytes the caller's header knew about are read; later fields keep their defaults.
  if (user->struct_size < offsetof(tf_inspect_opts, K) || user->struct_size > 4096)
    return tf::fail(TF_EINVAL, "tf_inspect: opts.struct_size is %zu: set it to sizeof(tf_inspect_opts)", user->struct_size);
  tf_inspect_opts given{};
  std::memcpy(&given, user, std::min(user->struct_size, sizeof(given)));
  given.struct_size = sizeof(given);
  user = &given;
  tf_inspect_opts o = given;
  if (o.op != TF_OP_SPMM_SPMM && o.op != TF_OP_GEMM_SPMM)
    return tf::fail(TF_EINVAL, "tf_inspect: unknown op %d", o.op);
  if (o.N <= 0) return tf::fail(TF_EINVAL, "tf_inspect: N must be positive");
  if (o.op == TF_OP_GEMM_SPMM) {
    if (o.K <= 0) return tf::fail(TF_EINVAL, "tf_inspect: GeMM-SpMM needs K > 0");
  } else {
    o.K = 0;
  }
  // The MFMA kernels take widths of 32, 64 .. 256 columns.  Any other N of a GeMM-SpMM is cut into equal
  // column panels of such a width (the last one padded with zero columns of C); the executor runs the
  // schedule once per panel.
  const int user_N = o.N;
  int n_panels = 1;
  if (o.op == TF_OP_GEMM_SPMM && (o.N % 32 != 0 || o.N > 256)) {
    n_panels = (o.N + 255) / 256;
    o.N = ((o.N + n_panels - 1) / n_panels + 31) / 32 * 32;
  }
  if ((long long)std::max(L, M) * o.N > INT_MAX)  // (the width the kernels see: a panel's, when N is cut into panels)
    return tf::fail(TF_EUNSUPPORTED, "tf_inspect: rows*N exceeds int32 indexing");
  // The MFMA kernels walk k in steps of 8: a K that is not a multiple of 8 is rounded up here and
  // the executor pads B's columns and C's rows with zeros into its workspace on every call.
  const int user_K = o.K;
  o.K = (o.K + 7) / 8 * 8;
  const bool has_inner = o.op == TF_OP_SPMM_SPMM && o.inner_Ap != nullptr;
  // GeMM-SpMM tiles keep C in registers when a wavefront's K x 16 slice (two slices when
  // N > 128) fits 64 registers per lane; LDS then holds only the slab, rows padded by 4 floats.
  const bool gemm_regw = o.op == TF_OP_GEMM_SPMM && o.K <= 256 &&
                         (o.K <= 64 ? 4 : o.K <= 128 ? 8 : 16) * (o.N > 128 ? 2 : 1) <= 16;
  // ... and stream: one workgroup per compute unit walks a long run of rows and keeps the last
  // ring_rows intermediate rows in LDS (a power of two, at least 256: 64 rows being written,
  // 64 of alignment slack and a reach of 128 or more).
  const int stream_fixed = 2 * 64 * 36 * 4 + ((o.K <= 128 && o.N <= 128) ? 8 : 4) * 64 * 8 + (1024 + 4) * 4;  // X staging + consumer scratch + step table (<= 1024 steps)
  auto ring_for = [&](int budget) {
    int r = 0;
    for (int c = 256; c <= 4096 && stream_fixed + (long long)c * (o.N + 4) * 4 <= budget; c *= 2) r = c;
    return r;
  };
  // (a run needs a hundred rows or more to pay for its start-up and halo: with fewer than 96 rows
  // per compute unit the tile kernel, which spreads over all of them, is the faster one --
  // banded matrix, K = N = 128: 16,384 rows 23 us in tiles / 27 us in runs, 24,576 rows 36 / 28)
  if (o.compute_units <= 0) o.compute_units = tf::default_compute_units();
  const bool long_enough = user->tile_rows > 0 || M >= 96LL * o.compute_units;
  const int ring_rows = gemm_regw && long_enough ? ring_for(o.lds_budget_bytes > 0 ? o.lds_budget_bytes : kMaxLds) : 0;
  const bool gemm_stream = ring_rows > 0;
  if (o.lds_budget_bytes <= 0)  // two workgroups per CU, except for the kernels that own a compute unit
    o.lds_budget_bytes = o.op == TF_OP_GEMM_SPMM ? (gemm_stream ? kMaxLds : gemm_regw ? 81920 : 131072)
                                                 : has_inner ? 81920 : 65536;
  if (o.lds_budget_bytes > kMaxLds)
    return tf::fail(TF_EINVAL, "tf_inspect: lds_budget_bytes %d exceeds %d", o.lds_budget_bytes, kMaxLds);
  // (recomputed GEMM rows cost MFMA time, unless the matrix is too short to fill the device anyway)
  if (o.max_redundancy <= 0.f) o.max_redundancy = (o.op == TF_OP_GEMM_SPMM && long_enough) ? 1.5f : 3.0f;
  if (o.max_redundancy < 1.f) o.max_redundancy = 1.f;
  if (o.long_row_nnz <= 0) o.long_row_nnz = 32;
  if (o.long_row_nnz > 2048) o.long_row_nnz = 2048;  // a row must fit one staging batch of the row kernel
  if (o.compute_units <= 0) o.compute_units = tf::default_compute_units();

  // LDS the tile GEMM needs for staging C, before any slab row.
  int gemm_kc = 0, staging = 0;
  if (gemm_regw) staging = 2 * 64 * 36 * 4;  // the two X staging buffers of the register-W tile kernel
  if (o.op == TF_OP_GEMM_SPMM && !gemm_regw) {
    const int stage_cap = std::min(32768, o.lds_budget_bytes / 2);
    gemm_kc = std::min(o.K, std::max(8, (stage_cap / (4 * o.N)) / 8 * 8));
    staging = gemm_kc * o.N * 4;
  }
  // (the register-W tile kernel also keeps 16 bytes per fused row behind the slab)
  const int row_bytes = gemm_regw ? (o.N + 4) * 4 + 16 : o.N * 4;
  const int p_max = (o.lds_budget_bytes - staging) / row_bytes;
  if (p_max < 8)
    return tf::fail(TF_EINVAL, "tf_inspect: LDS budget %d holds only %d intermediate rows of N=%d behind %d bytes of staging",
                    o.lds_budget_bytes, std::max(p_max, 0), o.N, staging);
  if (o.strip_cols <= 0) o.strip_cols = 32;
  if (o.strip_cols != 32 && o.strip_cols != 64)
    return tf::fail(TF_EINVAL, "tf_inspect: strip_cols must be 32 or 64");
  const bool have_inner = o.op == TF_OP_SPMM_SPMM && o.inner_Ap && (o.inner_Ai || o.inner_Ap[M] == 0) && o.inner_cols > 0;
  const bool want_window = have_inner && o.N % o.strip_cols == 0 && o.wide_strips <= 0;
  // (measured faster than the lane-group kernel from 1,024 to 2^20 rows of a band, so it is the
  // default wherever it applies)
  // (the kernel addresses the CSR arrays with 32-bit byte offsets and loads four entries at a time)
  const bool want_wide = have_inner && o.N % 64 == 0 && o.inner_Ap[M] >= 4 && nnz >= 4 && o.inner_Ap[M] < (1 << 30) && nnz < (1 << 30) &&
                         (o.wide_strips > 0 || (o.wide_strips == 0 && user->strip_cols <= 0 && user->lds_budget_bytes <= 0 &&
                                              user->tile_rows <= 0));
  int r_cap = o.tile_rows > 0 ? o.tile_rows : ceil_div(M, 2 * o.compute_units);
  if (o.op == TF_OP_GEMM_SPMM) r_cap = ceil_div(r_cap, 32) * 32;
  r_cap = std::max(r_cap, o.tile_rows > 0 ? 1 : 64);  // smaller tiles spend most of their work on halo rows
  r_cap = std::min(r_cap, p_max);
  o.tile_rows = r_cap;

  auto *S = new (std::nothrow) tf_schedule();
  if (!S) return tf::fail(TF_ENOMEM, "tf_inspect: out of host memory");
  try {
    S->opts = o;
    S->opts.inner_Ap = nullptr;  // the caller's arrays are not kept
    S->opts.inner_Ai = nullptr;
    S->L = L;
    S->M = M;
    S->nnz = nnz;
    S->pattern_hash = tf_pattern_hash(L, Ap, Ai);
    S->gemm_kc = gemm_kc;
    S->user_K = user_K;
    S->user_N = user_N;
    S->n_panels = n_panels;
    S->gemm_regw = gemm_regw;
    S->gemm_stream = gemm_stream;
    S->ring_rows = ring_rows;
    S->slab_ld = gemm_regw ? o.N + 4 : o.N;

    // Column extent of every second-op row (columns need not be sorted).
    std::vector<int> lo(L), hi(L);
    for (int i = 0; i < L; ++i) {
      int a = INT_MAX, b = -1;
      for (int k = Ap[i]; k < Ap[i + 1]; ++k) {
        const int c = Ai[k];
        if (c < 0 || c >= M) {
          delete S;
          return tf::fail(TF_EINVAL, "tf_inspect: column %d out of range at row %d", c, i);
        }
        a = std::min(a, c);
        b = std::max(b, c);
      }
      if (b < 0) { a = std::min(i, M - 1); b = a - 1; }  // empty row: no dependence
      lo[i] = a;
      hi[i] = b + 1;
    }
    std::vector<char> fused(L, 0);

    // ---- windowed tiles (SpMM-SpMM with a known inner pattern) -------------------------
    // Every row must fuse, and the rows of C that a tile's producer rows read must form a
    // window small enough to sit in LDS next to the slab, one strip of columns at a time.
    // Two kernels run such tiles.  Wide strips: 64 columns at a time, LDS holds the window,
    // the slab and the row pointers, the entries are read from the CSR arrays in place, and
    // one workgroup of 1024 threads owns a compute unit and all of its LDS (a tile per compute
    // unit: long matrices).  Narrow strips: 32 or 64 columns, the tile's entries staged in LDS
    // as well, two workgroups per compute unit.
    bool windowed = false, win_wide = false;
    auto build_window = [&](bool wide, int wide_cap = 0) {
      const int *Bp = o.inner_Ap, *Bi = o.inner_Ai;
      const int SW = wide ? 64 : o.strip_cols;
      const int budget = wide ? (user->lds_budget_bytes > 0 ? user->lds_budget_bytes : kMaxLds) : o.lds_budget_bytes;
      const int cap = wide ? (wide_cap > 0 ? wide_cap : user->tile_rows > 0 ? user->tile_rows : std::max(64, ceil_div(M, o.compute_units))) : r_cap;
      std::vector<int> blo(M), bhi(M);
      bool ok = (Bp[0] == 0);
      for (int r = 0; r < M && ok; ++r) {
        int a = INT_MAX, b = -1;
        if (Bp[r + 1] < Bp[r]) { ok = false; break; }
        for (int k = Bp[r]; k < Bp[r + 1]; ++k) {
          const int c = Bi[k];
          if (c < 0 || c >= o.inner_cols) { ok = false; break; }
          a = std::min(a, c);
          b = std::max(b, c);
        }
        blo[r] = a;      // INT_MAX / 0 for an empty row: no constraint
        bhi[r] = b + 1;
      }
      auto a16 = [](long long x) { return (x + 15) / 16 * 16; };
      auto lds_of = [&](int P, int R, long long nz, int Wc) {
        if (wide) return a16(4LL * (P + 1)) + a16(4LL * (R + 1)) + 4LL * SW * ((long long)Wc + P);
        return a16(4LL * (P + 1)) + a16(4LL * R) + a16(8LL * (nz + 2LL * P)) + 4LL * SW * ((long long)Wc + P);  // 2 = pad slots per staged row
      };
      std::vector<tf::TileDesc> tiles;
      std::vector<int> ids, win;
      long long prod_rows = 0;
      int lds_max = 0, slab = 0;
      int s = 0;
      while (ok && s < M) {
        int wlo = s, whi = s, clo = INT_MAX, chi = 0, e = s;
        while (e < M && e - s < cap) {
          int nlo = std::min(wlo, e), nhi = std::max(whi, e + 1);
          if (e < L) { nlo = std::min(nlo, lo[e]); nhi = std::max(nhi, hi[e]); }
          int nclo = clo, nchi = chi;
          for (int r = nlo; r < wlo; ++r) { nclo = std::min(nclo, blo[r]); nchi = std::max(nchi, bhi[r]); }
          for (int r = std::max(whi, nlo); r < nhi; ++r) { nclo = std::min(nclo, blo[r]); nchi = std::max(nchi, bhi[r]); }
          const int Wc = nchi > nclo ? nchi - nclo : 0;
          if (lds_of(nhi - nlo, e + 1 - s, (long long)Bp[nhi] - Bp[nlo], Wc) > budget) break;
          wlo = nlo; whi = nhi; clo = nclo; chi = nchi; ++e;
        }
        // (the last tile of the matrix may be short, and then has relatively more halo: 1.5x the limit)
        if (e == s || (e != M && e - s < std::min(cap, 16)) ||
            (float)(whi - wlo) > (e == M ? 1.5f : 1.0f) * o.max_redundancy * (float)(e - s)) { ok = false; break; }
        tf::TileDesc t{};
        t.own_begin = s; t.own_end = e; t.prod_begin = wlo; t.prod_end = whi;
        t.wb_begin = t.wb_end = s;
        t.cons_begin = (int)ids.size();
        for (int i = s; i < e && i < L; ++i) ids.push_back(i);
        t.cons_end = (int)ids.size();
        if (chi <= clo) { clo = 0; chi = 0; }
        win.push_back(clo); win.push_back(chi);
        lds_max = std::max<long long>(lds_max, lds_of(whi - wlo, e - s, (long long)Bp[whi] - Bp[wlo], chi - clo));
        slab = std::max(slab, whi - wlo);
        prod_rows += whi - wlo;
        tiles.push_back(t);
        s = e;
      }
      if (!(ok && L <= M)) return false;
      S->inner_nnz = Bp[M];
      if (!S->inner_hash) S->inner_hash = (Bp == Ap && Bi == Ai && L == M) ? S->pattern_hash : tf_pattern_hash(M, Bp, Bi);
      S->tiles.swap(tiles);
      S->fused_ids.swap(ids);
      S->win.swap(win);
      S->n_producer_rows = prod_rows;
      S->slab_rows = slab;
      S->lds_bytes = lds_max;
      S->opts.strip_cols = SW;
      S->opts.tile_rows = cap;
      std::fill(fused.begin(), fused.end(), 1);
      return true;
    };
    if (want_wide) windowed = win_wide = build_window(true);
    if (win_wide && user->tile_rows <= 0 && (int)S->tiles.size() > o.compute_units) {
      // More tiles than compute units (LDS, not the row count, set the tile size): every compute
      // unit takes several tiles in turn, so size them for a whole number of turns.
      auto keep_tiles = S->tiles; auto keep_ids = S->fused_ids; auto keep_win = S->win;
      const long long keep_prod = S->n_producer_rows; const int keep_slab = S->slab_rows, keep_lds = S->lds_bytes;
      const int first_turns = ceil_div((int)S->tiles.size(), o.compute_units);
      bool done = (int)S->tiles.size() == o.compute_units * first_turns;
      for (int turns = first_turns; !done && turns <= first_turns + 2; ++turns) {
        const int cap2 = ceil_div(M, o.compute_units * turns);
        if (cap2 < 64) break;
        done = build_window(true, cap2) && (int)S->tiles.size() <= o.compute_units * turns &&
               (int)S->tiles.size() > o.compute_units * (turns - 1) + o.compute_units / 2;
      }
      if (!done) {  // (keeps the first tiling)
        S->tiles.swap(keep_tiles); S->fused_ids.swap(keep_ids); S->win.swap(keep_win);
        S->n_producer_rows = keep_prod; S->slab_rows = keep_slab; S->lds_bytes = keep_lds;
        S->opts.tile_rows = std::max(64, ceil_div(M, o.compute_units));
      }
    }
    if (!windowed && want_window) windowed = build_window(false);
    S->win_wide = win_wide;
    S->windowed = windowed;
    if (!windowed) S->opts.strip_cols = 0;

    // ---- marching runs (stencils on 3D grids: no range of consecutive rows holds a row's dependences) ----
    if (!windowed && have_inner && o.march >= 0) {
      if (tf::build_march(S, M, Ap, Ai, o.inner_Ap, o.inner_Ai, o, given)) {
        *out = S;
        return TF_OK;
      }
      if (o.march > 0) {
        delete S;
        return tf::fail(TF_EUNSUPPORTED, "tf_inspect: no marching schedule for this pattern (needs a square matrix with at most 32 entries "
                        "per row in both patterns, N a multiple of 64, a grid given or found, and a column of grid points whose rows fit LDS)");
      }
    }

    // A row whose own reach (itself plus its columns) exceeds the slab can never fuse.
    auto reach_lo = [&](int i) { return std::min(lo[i], std::min(i, M - 1)); };
    auto reach_hi = [&](int i) { return std::max(hi[i], std::min(i, M - 1) + 1); };
    auto never = [&](int i) { return reach_hi(i) - reach_lo(i) > p_max; };

    int slab_rows = windowed ? S->slab_rows : 0;
    int s = windowed ? M : 0;

    // ---- streamed runs (GeMM-SpMM, C in registers) ----------------------------------------
    // One run per compute unit.  A run produces the rows [prod_begin, prod_end) in steps of 64
    // and keeps the last ring_rows of them; a fused row is computed during the step after the
    // one that produced its last column, and by then its first column must still be in the
    // ring: with q(c) = (c - prod_begin) / 64 that is q(last) - q(first) <= ring_rows/64 - 2.
    if (gemm_stream) {
      int own = user->tile_rows > 0 ? std::max(user->tile_rows, 64)
                                     : std::max(ceil_div(M, o.compute_units), 128);  // one run per compute unit: a run
      // count that leaves compute units idle costs more than short runs do (32,768 rows: 29 us in 256 runs of 128, 43 us in 128 of 256)
      own = std::min(own, 1000 * 64 - 2 * ring_rows);  // a run's step table holds 1024 steps
      const int qspan = ring_rows / 64 - 2;
      // What the consumer wavefronts of the kernel take per step without falling behind, and
      // the longest row a lane group holds in registers.
      const int lpr = o.N <= 32 ? 8 : o.N <= 64 ? 16 : 32;
      const int per_round = ((o.K <= 128 ? 8 : 4) * 64 / lpr) * ((o.K <= 64 ? 4 : o.K <= 128 ? 8 : 16) / 2);
      const int step_cap = per_round * ceil_div(64, per_round);  // lane groups x intervals x rows per interval
      const int max_len = 32;
      S->stream_step_cap = step_cap;
      S->stream_max_len = max_len;
      // without a run length from the caller the rows are dealt evenly: M / own runs, one per compute unit
      const int n_even = user->tile_rows > 0 ? 0 : std::max({1, std::min(o.compute_units, M / 128), ceil_div(M, own)});
      int run = 0;
      while (s < M) {
        int e = n_even > 0 ? (int)((long long)(run + 1) * M / n_even) : std::min(M, s + own);
        ++run;
        if (n_even == 0 && M - e < own / 2) e = M;  // a short last run would be mostly halo: the one before takes its rows
        tf::TileDesc t{};
        t.own_begin = s; t.own_end = e; t.prod_begin = s; t.prod_end = e;
        t.cons_begin = t.cons_end = (int)S->fused_ids.size();
        t.wb_begin = t.wb_end = s;
        int hlo = INT_MAX, hhi = -1, useful = 0;
        auto candidate = [&](int i) {
          return Ap[i + 1] > Ap[i] && Ap[i + 1] - Ap[i] <= max_len && hi[i] - lo[i] <= ring_rows - 64 &&
                 lo[i] >= s - ring_rows && hi[i] <= e + ring_rows;
        };
        for (int i = s; i < e && i < L; ++i)
          if (candidate(i)) { hlo = std::min(hlo, lo[i]); hhi = std::max(hhi, hi[i]); }
        if (hhi > hlo) {
          const int pb = std::min(hlo, s), pe = std::max(hhi, e);
          const int steps = ceil_div(pe - pb, 64);
          std::vector<std::vector<int>> by_step(steps + 1);
          for (int i = s; i < e && i < L; ++i) {
            if (!candidate(i)) continue;
            const int qf = (lo[i] - pb) / 64, ql = (hi[i] - 1 - pb) / 64;
            if (ql - qf <= qspan) { by_step[ql + 1].push_back(i); ++useful; }
          }
          if (4 * useful >= e - s && (float)(steps * 64) <= o.max_redundancy * (float)std::max(e - s, 64)) {
            t.prod_begin = pb; t.prod_end = pe;
            S->tile_step.push_back((int)S->step_ptr.size());
            // A step takes at most step_cap rows; the rest wait for the next step if their first
            // column is still in the ring then, and are left to the remainder otherwise.  The
            // step after the last production step takes everything.
            std::vector<int> carry, next;
            for (int q = 0; q <= steps; ++q) {
              S->step_ptr.push_back((int)S->fused_ids.size());
              int taken = 0;
              next.clear();
              auto place = [&](int i) {
                if (taken < step_cap || q == steps) { S->fused_ids.push_back(i); fused[i] = 1; ++taken; }
                else if ((lo[i] - pb) / 64 >= q + 1 - ring_rows / 64 + 1) next.push_back(i);
              };
              for (int i : carry) place(i);
              for (int i : by_step[q]) place(i);
              carry.swap(next);
            }
            S->step_ptr.push_back((int)S->fused_ids.size());
            t.cons_end = (int)S->fused_ids.size();
            slab_rows = std::max(slab_rows, pe - pb);
          }
        }
        if ((int)S->tile_step.size() == (int)S->tiles.size()) S->tile_step.push_back(-1);  // nothing streamed here
        S->n_producer_rows += t.prod_end - t.prod_begin;
        S->tiles.push_back(t);
        s = e;
      }
      S->fused_rec.reserve(4 * S->fused_ids.size());
      for (int i : S->fused_ids) {
        S->fused_rec.push_back(i); S->fused_rec.push_back(Ap[i]); S->fused_rec.push_back(Ap[i + 1]); S->fused_rec.push_back(0);
      }
    }
    while (s < M) {
      tf::TileDesc t{};
      // 1. grow a tile whose producer window covers every fusable row it owns
      int wlo = s, whi = s, e = s;
      while (e < M && e - s < r_cap) {
        int nlo = std::min(wlo, e), nhi = std::max(whi, e + 1);
        if (e < L && !never(e)) { nlo = std::min(nlo, lo[e]); nhi = std::max(nhi, hi[e]); }
        if (nhi - nlo > p_max) break;
        wlo = nlo; whi = nhi; ++e;
      }
      const bool halo_ok = (e > s) && (e == M || e - s >= std::min(r_cap, 16)) &&
                           (float)(whi - wlo) <= (e == M ? 1.5f : 1.0f) * o.max_redundancy * (float)(e - s);
      t.cons_begin = (int)S->fused_ids.size();
      if (halo_ok) {
        t.own_begin = s; t.own_end = e; t.prod_begin = wlo; t.prod_end = whi;
        for (int i = s; i < e && i < L; ++i)
          if (!never(i)) { S->fused_ids.push_back(i); fused[i] = 1; }
      } else {
        // 2. the reference's tiling: no recomputation, rows fuse iff their columns are in the tile
        e = std::min(M, s + r_cap);
        t.own_begin = s; t.own_end = e; t.prod_begin = s; t.prod_end = e;
        for (int i = s; i < e && i < L; ++i)
          if (lo[i] >= s && hi[i] <= e) { S->fused_ids.push_back(i); fused[i] = 1; }
      }
      t.cons_end = (int)S->fused_ids.size();
      {  // rows without entries fuse trivially; a tile that would fuse only such rows fuses nothing
        // and one that would fuse less than a quarter of its rows is not worth a workgroup of its own
        int useful = 0;
        for (int q = t.cons_begin; q < t.cons_end; ++q)
          useful += Ap[S->fused_ids[q] + 1] > Ap[S->fused_ids[q]];
        if (4 * useful < t.own_end - t.own_begin) {
          for (int q = t.cons_begin; q < t.cons_end; ++q) fused[S->fused_ids[q]] = 0;
          S->fused_ids.resize(t.cons_begin);
          t.cons_end = t.cons_begin;
        }
      }
      if (t.cons_end > t.cons_begin) slab_rows = std::max(slab_rows, t.prod_end - t.prod_begin);
      else { t.prod_begin = t.own_begin; t.prod_end = t.own_end; }  // nothing to fuse: no halo
      t.wb_begin = t.wb_end = t.own_begin;
      S->n_producer_rows += t.prod_end - t.prod_begin;
      S->tiles.push_back(t);
      s = e;
    }

    // Remainder: rows not fused; long ones are cut into chunks of up to chunk_nnz entries, each
    // worked on by a whole workgroup.
    const int chunk_nnz = std::max(o.long_row_nnz, 1024);
    std::vector<char> need(M, 0);
    for (int i = 0; i < L; ++i) {
      if (fused[i]) { S->fused_nnz += Ap[i + 1] - Ap[i]; continue; }
      for (int k = Ap[i]; k < Ap[i + 1]; ++k) need[Ai[k]] = 1;
      const int len = Ap[i + 1] - Ap[i];
      if (len > o.long_row_nnz) {
        tf::LongRow lr{i, (int)S->long_chunks.size(), 0, 0};
        for (int k = Ap[i]; k < Ap[i + 1]; k += chunk_nnz) {
          tf::LongChunk c{i, k, std::min(Ap[i + 1], k + chunk_nnz), (int)S->long_chunks.size()};
          S->long_chunks.push_back(c);
          ++lr.count;
        }
        S->long_rows.push_back(lr);
      } else {
        S->rem_rows.push_back(i);
      }
    }
    // Long rows by column.  On a power-law graph a few intermediate rows take most of the reads
    // of the long rows, but not few enough to survive in an L2 next to the stream of all the
    // others.  Each of the 8 XCDs has its own L2: the most-read rows are dealt to 8 partitions
    // that fit one L2 each, every long row's entries are regrouped by partition (CSR order kept
    // inside a group), and a group is worked on, like a short row, by the XCD of its partition;
    // entries outside all partitions ("cold") go to all XCDs as before.  Groups are cut into
    // segments of at most 64 entries; a row's segments are added up in a fixed order.
    std::vector<signed char> part;  // per intermediate row: its hot partition, or -1 (empty without long_part)
    {
      long long long_nnz = 0;
      for (const auto &lr : S->long_rows) long_nnz += Ap[lr.row + 1] - Ap[lr.row];
      const bool want = o.long_row_partition > 0 ||
                        (o.long_row_partition == 0 && long_nnz >= (1 << 20) && (long long)M * o.N * 4 > (64LL << 20));
      // (three times an L2's 4 MB measured best on the R-MAT graph: 2.68 ms per step with 4 MB, 2.54 with 12 or
      // 16 MB, 2.60 with 32 MB -- the reads inside a partition are skewed too, and its hottest rows are what stays)
      const int part_rows = std::max(64, (o.hot_partition_bytes > 0 ? o.hot_partition_bytes : (12 << 20)) / (o.N * 4));
      // Regrouped rows pay for their partial sums (a row of 4N bytes written and read again per group): with the
      // threshold left to the library, rows of up to 64 entries stay whole rows of the row kernel (measured on the
      // 2^21-node R-MAT step, thresholds 32 / 40 / 48 / 64 / 96: 2.04 / 1.97 / 1.97 / 1.96 / 1.97 ms).
      if (want && user->long_row_nnz <= 0 && S->long_chunks.size() < (size_t)INT_MAX) {
        constexpr int kPartitionedFrom = 64;
        std::vector<tf::LongRow> keep_rows;
        std::vector<tf::LongChunk> keep_chunks;
        for (const auto &lr : S->long_rows) {
          if (Ap[lr.row + 1] - Ap[lr.row] <= kPartitionedFrom) { S->rem_rows.push_back(lr.row); continue; }
          tf::LongRow nr{lr.row, (int)keep_chunks.size(), lr.count, 0};
          for (int c = 0; c < lr.count; ++c) {
            tf::LongChunk ch = S->long_chunks[lr.first + c];
            ch.slot = (int)keep_chunks.size();
            keep_chunks.push_back(ch);
          }
          keep_rows.push_back(nr);
        }
        S->long_rows.swap(keep_rows);
        S->long_chunks.swap(keep_chunks);
        std::sort(S->rem_rows.begin(), S->rem_rows.end());
        S->opts.long_row_nnz = o.long_row_nnz = kPartitionedFrom;
        long_nnz = 0;
        for (const auto &lr : S->long_rows) long_nnz += Ap[lr.row + 1] - Ap[lr.row];
      }
      if (want && !S->long_rows.empty() && long_nnz < INT_MAX) {
        constexpr int kParts = 8, kSegMax = 64, kPad = 256, kMinGroup = 4;
        std::vector<int> reads(M, 0);
        for (const auto &lr : S->long_rows)
          for (int k = Ap[lr.row]; k < Ap[lr.row + 1]; ++k) ++reads[Ai[k]];
        std::vector<int> hot;
        for (int c = 0; c < M; ++c)
          if (reads[c] >= 2) hot.push_back(c);
        const size_t n_hot = std::min(hot.size(), (size_t)kParts * part_rows);
        std::partial_sort(hot.begin(), hot.begin() + n_hot, hot.end(),
                          [&](int a, int b) { return reads[a] != reads[b] ? reads[a] > reads[b] : a < b; });
        hot.resize(n_hot);
        part.assign(M, -1);
        for (size_t h = 0; h < n_hot; ++h) {  // dealt in turn, snake-wise, so that the partitions' read counts match
          const int lap = (int)(h / kParts), pos = (int)(h % kParts);
          part[hot[h]] = (signed char)((lap & 1) ? kParts - 1 - pos : pos);
        }
        // segments per class (0..7 hot, 8 cold), in row order
        std::vector<std::vector<int>> cls_ptr(kParts + 1), cls_src(kParts + 1);
        std::vector<std::vector<std::pair<int, int>>> row_segs(S->long_rows.size());  // (class, index in class)
        for (auto &v : cls_ptr) v.push_back(0);
        std::vector<int> bucket[kParts + 1];
        for (size_t r = 0; r < S->long_rows.size(); ++r) {
          const int i = S->long_rows[r].row;
          for (auto &b : bucket) b.clear();
          for (int k = Ap[i]; k < Ap[i + 1]; ++k) bucket[part[Ai[k]] < 0 ? kParts : part[Ai[k]]].push_back(k);
          // a handful of entries does not pay for a partial sum of its own: such groups join the cold one
          bool moved = false;
          for (int c = 0; c < kParts; ++c)
            if (!bucket[c].empty() && (int)bucket[c].size() < kMinGroup) {
              bucket[kParts].insert(bucket[kParts].end(), bucket[c].begin(), bucket[c].end());
              bucket[c].clear();
              moved = true;
            }
          if (moved) std::sort(bucket[kParts].begin(), bucket[kParts].end());
          for (int c = 0; c <= kParts; ++c)
            for (size_t b0 = 0; b0 < bucket[c].size(); b0 += kSegMax) {
              const size_t b1 = std::min(bucket[c].size(), b0 + kSegMax);
              cls_src[c].insert(cls_src[c].end(), bucket[c].begin() + b0, bucket[c].begin() + b1);
              row_segs[r].emplace_back(c, (int)cls_ptr[c].size() - 1);
              cls_ptr[c].push_back((int)cls_src[c].size());
            }
        }
        size_t per = 0;
        for (int c = 0; c < kParts; ++c) per = std::max(per, cls_ptr[c].size() - 1);
        per = (per + kPad - 1) / kPad * kPad;  // whole workgroups of the row kernel, whatever its rows per workgroup
        const size_t n_cold = cls_ptr[kParts].size() - 1;
        if ((long long)kParts * per + n_cold < INT_MAX / 2) {
          S->long_part = true;
          S->seg_per_xcd = (int)per;
          S->hot_cols = (int)n_hot;
          S->long_chunks.clear();
          S->seg_ptr.assign(1, 0);
          std::vector<int> cls_base(kParts + 1);
          for (int c = 0; c <= kParts; ++c) {
            cls_base[c] = (int)S->seg_ptr.size() - 1;
            const int base = (int)S->seg_src.size();
            S->seg_src.insert(S->seg_src.end(), cls_src[c].begin(), cls_src[c].end());
            for (size_t q = 1; q < cls_ptr[c].size(); ++q) S->seg_ptr.push_back(base + cls_ptr[c][q]);
            if (c < kParts)
              for (size_t q = cls_ptr[c].size() - 1; q < per; ++q) S->seg_ptr.push_back(S->seg_ptr.back());  // empty pads
          }
          S->seg_col.resize(S->seg_src.size());
          for (size_t k = 0; k < S->seg_src.size(); ++k) S->seg_col[k] = Ai[S->seg_src[k]];
          // the executor copies A's values into this order walking A's array once: pairs sorted by source
          {
            std::vector<int> pos_of((size_t)nnz);
            for (size_t e = 0; e < S->seg_src.size(); ++e) pos_of[S->seg_src[e]] = (int)e;
            S->ent_src.reserve(S->seg_src.size());
            S->ent_pos.reserve(S->seg_src.size());
            std::vector<int> lrows;
            for (const auto &lr : S->long_rows) lrows.push_back(lr.row);
            std::sort(lrows.begin(), lrows.end());
            for (const int i : lrows)
              for (int k = Ap[i]; k < Ap[i + 1]; ++k) { S->ent_src.push_back(k); S->ent_pos.push_back(pos_of[k]); }
          }
          // A row adds up its segments' sums in a fixed order; a hub row has thousands of them, so
          // groups of up to 32 segments are summed first (into slots behind the segments').
          const int n_seg = (int)S->seg_ptr.size() - 1;
          constexpr int kGroup = 32;
          std::vector<int> slots;
          for (size_t r = 0; r < S->long_rows.size(); ++r) {
            slots.clear();
            for (const auto &cs : row_segs[r]) slots.push_back(cls_base[cs.first] + cs.second);
            if ((int)slots.size() > kGroup) {
              std::vector<int> groups;
              for (size_t b0 = 0; b0 < slots.size(); b0 += kGroup) {
                const size_t b1 = std::min(slots.size(), b0 + kGroup);
                tf::LongRow g{n_seg + (int)S->seg_groups.size(), (int)S->lrow_seg.size(), (int)(b1 - b0), 0};
                S->lrow_seg.insert(S->lrow_seg.end(), slots.begin() + b0, slots.begin() + b1);
                groups.push_back(g.row);
                S->seg_groups.push_back(g);
              }
              slots.swap(groups);
            }
            S->long_rows[r].first = (int)S->lrow_seg.size();
            S->long_rows[r].count = (int)slots.size();
            S->lrow_seg.insert(S->lrow_seg.end(), slots.begin(), slots.end());
          }
        }
      }
    }
    // Remainder rows of similar length go together: a lane group walks a row alone, so a
    // workgroup is as slow as its longest row.  Order is kept inside a length class, and a
    // matrix whose rows all fall in one class keeps its order entirely.
    {
      auto cls = [&](int i) {
        const int len = Ap[i + 1] - Ap[i];
        return len <= 8 ? 0 : len <= 32 ? 1 : len <= 128 ? 2 : len <= 512 ? 3 : 4;
      };
      std::vector<int> byc[5];
      // Rows without entries, when they are many (half of the nodes of an R-MAT graph are isolated), leave
      // the list: a row of zeros needs no lane group and no row pointers, a fill kernel over the rows'
      // own list writes it (the row kernel of the 2^21-node R-MAT step: 0.69 -> 0.50 ms, the fill 0.12 ms).
      {
        size_t n_empty = 0;
        for (int i : S->rem_rows) n_empty += Ap[i + 1] == Ap[i];
        if (n_empty >= 4096 && n_empty * 8 >= S->rem_rows.size()) {
          std::vector<int> keep;
          keep.reserve(S->rem_rows.size() - n_empty);
          S->zero_rows.reserve(n_empty);
          for (int i : S->rem_rows) (Ap[i + 1] == Ap[i] ? S->zero_rows : keep).push_back(i);
          S->rem_rows.swap(keep);
        }
      }
      for (int i : S->rem_rows) byc[cls(i)].push_back(i);
      S->rem_rows.clear();
      for (auto &v : byc) S->rem_rows.insert(S->rem_rows.end(), v.begin(), v.end());
      S->rem_identity = (int)S->rem_rows.size() == L;
      for (int q = 0; q < L && S->rem_identity; ++q) S->rem_identity = (S->rem_rows[q] == q);
      // Reordered adjacency (createReorderedAdj, GCN_Single_Layer_SP_Demo_Utils.h:618-653): a list that is
      // not simply all rows in order gets its rows stored side by side in list order, so that a
      // workgroup reads one stretch of columns and values instead of one stretch per row.
      if (!S->rem_identity && !S->rem_rows.empty() && o.reorder_adjacency >= 0) {
        S->rem_ptr.reserve(S->rem_rows.size() + 1);
        S->rem_ptr.push_back(0);
        for (int i : S->rem_rows) {
          for (int k = Ap[i]; k < Ap[i + 1]; ++k) { S->rem_col.push_back(Ai[k]); S->rem_src.push_back(k); }
          S->rem_ptr.push_back((int)S->rem_col.size());
        }
        // Gathers that are not expected to find their row in L2 are marked (top bit of the column): the row kernel
        // fetches those with streaming loads, so that they do not push out the rows that have readers.  On a
        // power-law graph the short rows read the same few hub rows as everybody else (the 16,384 most-read rows
        // take half of their reads on the 2^21-node R-MAT graph) next to a stream of rows read once; left
        // alone, that stream leaves an L2 hit rate under a quarter.  Which XCD a row runs on cannot help here as it
        // does for the long rows' segments: a short row's few columns are spread over all partitions
        // (measured on that step: the rows' launch 0.495 -> 0.45 ms with 8 MB of unmarked rows; 4 MB 0.52, 16 MB 0.47 -- and, once the
        // intermediate's rows lie in the order of their reads, 8 / 16 / 32 / 64 MB: 0.419 / 0.393 / 0.388 / 0.386 ms).
        {
          const int want = o.short_row_hot_bytes;
          const long long bytes = want > 0 ? want : (want == 0 && S->long_part ? (32 << 20) : 0);
          const size_t keep_n = (size_t)(bytes / ((long long)o.N * 4));
          if (keep_n > 0 && o.N % 4 == 0) {
            std::vector<int> reads(M, 0), order;
            for (int c : S->rem_col) ++reads[c];
            for (int c = 0; c < M; ++c)
              if (reads[c] >= 2) order.push_back(c);
            const size_t nh = std::min(order.size(), keep_n);
            std::partial_sort(order.begin(), order.begin() + nh, order.end(),
                              [&](int a, int b) { return reads[a] != reads[b] ? reads[a] > reads[b] : a < b; });
            long long covered = 0;
            for (size_t h = 0; h < nh; ++h) covered += reads[order[h]];
            // (a set that takes less than a quarter of the reads is no hot set: an Erdos-Renyi graph has none)
            if (nh > 0 && covered * 4 >= (long long)S->rem_col.size()) {
              std::vector<char> is_hot(M, 0);
              for (size_t h = 0; h < nh; ++h) is_hot[order[h]] = 1;
              for (int &c : S->rem_col)
                if (!is_hot[c]) c |= INT_MIN;
              S->rem_flagged = true;
              S->rem_hot_rows = (int)nh;
            }
          }
        }
      }
    }

    // Row kernels: workgroup ids go to the XCDs round-robin, which keeps all eight of them in the
    // same neighbourhood of memory (measured faster than giving each XCD a far-away run of its
    // own, R-MAT: -18 %).  A caller may still ask for chunks of rows per XCD, or for one run each.
    S->xcd_chunk_rows = o.xcd_chunk_rows;

    // Tiles that fuse nothing are not launched as tiles: the intermediate rows they own go to
    // the row kernels (plain SpMM / GEMM), and only those some remainder row reads.  A GEMM
    // whose weight does not fit LDS has no row-list form; such tiles stay tiles.
    const bool plain_ok = o.op == TF_OP_SPMM_SPMM || (long long)o.K * o.N * 4 <= 131072;
    for (auto &t : S->tiles) {
      int a = -1, b = -1, cnt = 0;
      for (int r = t.own_begin; r < t.own_end; ++r)
        if (need[r]) { if (a < 0) a = r; b = r + 1; ++cnt; }
      if (a >= 0) { t.wb_begin = a; t.wb_end = b; }
      const bool fuses = t.cons_end > t.cons_begin;
      if (fuses || !plain_ok) {
        S->launch_tiles.push_back(t);
        if (gemm_stream) S->launch_step.push_back(S->tile_step[&t - S->tiles.data()]);
        if (a >= 0) S->n_writeback_rows += b - a;
      } else {
        for (int r = t.own_begin; r < t.own_end; ++r)
          if (need[r]) S->plain_rows.push_back(r);
        S->n_writeback_rows += cnt;
      }
    }
    // With column-partitioned long rows the rows of the hot partitions come first in the list: the
    // executor produces them first and starts the hot segments beside the rest of the GEMM.  (Only
    // when every hot row is a plain row: a hot row stored by a fused tile is ready even earlier.)
    if (S->long_part && o.op == TF_OP_GEMM_SPMM && !S->plain_rows.empty()) {
      auto mid = std::stable_partition(S->plain_rows.begin(), S->plain_rows.end(), [&](int r) { return part[r] >= 0; });
      S->plain_hot = (int)(mid - S->plain_rows.begin());
      if (S->plain_hot == (int)S->plain_rows.size()) S->plain_hot = 0;  // nothing left to run beside them
    }
    // The intermediate in the order in which it is read.  When nothing fuses, the step is a GEMM of the rows that are
    // read into HBM and gathers out of it through this schedule's own lists (rows in list order, long-row segments):
    // where a row of the intermediate lies is then the schedule's to choose.  The rows of the hot partitions come
    // first, partition by partition, then the others, each group by falling number of reads -- the rows that are
    // gathered most lie side by side (fewer pages under the gathers that miss, one stretch per XCD for those that
    // hit) and the rows nobody reads take no room in between.  Measured on the 2^21-node R-MAT step with the
    // columns of A renumbered by hand in this order: 2.10 -> 2.03 ms.
    if (o.op == TF_OP_GEMM_SPMM && S->launch_tiles.empty() && !S->plain_rows.empty() && S->long_chunks.empty() &&
        (S->rem_rows.empty() || !S->rem_ptr.empty()) && o.place_intermediate >= 0) {
      std::vector<int> treads(M, 0);
      for (int k = 0; k < Ap[L]; ++k) ++treads[Ai[k]];
      auto by_reads = [&](int a, int b) { return treads[a] != treads[b] ? treads[a] > treads[b] : a < b; };
      if (S->plain_hot > 0) {
        std::stable_sort(S->plain_rows.begin(), S->plain_rows.begin() + S->plain_hot,
                         [&](int a, int b) { return part[a] != part[b] ? part[a] < part[b] : by_reads(a, b); });
        std::stable_sort(S->plain_rows.begin() + S->plain_hot, S->plain_rows.end(), by_reads);
      } else if (S->long_part) {
        // (every hot row is a plain row here, or the hot rows are all of them: keep the partitions together)
        std::stable_sort(S->plain_rows.begin(), S->plain_rows.end(), [&](int a, int b) {
          const int pa = part[a] >= 0 ? part[a] : INT_MAX, pb = part[b] >= 0 ? part[b] : INT_MAX;
          return pa != pb ? pa < pb : by_reads(a, b);
        });
      } else {
        std::stable_sort(S->plain_rows.begin(), S->plain_rows.end(), by_reads);
      }
      S->t_pos.assign(M, -1);
      for (size_t q = 0; q < S->plain_rows.size(); ++q) S->t_pos[S->plain_rows[q]] = (int)q;
      bool ok = true;
      for (int c : S->rem_col) ok = ok && S->t_pos[c & INT_MAX] >= 0;
      for (int c : S->seg_col) ok = ok && S->t_pos[c & INT_MAX] >= 0;
      if (ok) {
        for (int &c : S->rem_col) c = S->t_pos[c & INT_MAX] | (c & INT_MIN);
        for (int &c : S->seg_col) c = S->t_pos[c & INT_MAX] | (c & INT_MIN);
      } else {
        S->t_pos.clear();  // (a column no list row was made for: leave everything where it was)
      }
    }
    S->slab_rows = slab_rows;
    S->lds_bytes_general = gemm_stream ? stream_fixed + ring_rows * (o.N + 4) * 4 : slab_rows * row_bytes + staging;
    if (!windowed) S->lds_bytes = S->lds_bytes_general;

    // Tiles that carry their rows through two layers, for when this is the second layer's schedule of
    // tf_gcn_two_layers (hidden width = this K, output width = this N).
    if (o.op == TF_OP_GEMM_SPMM && L == M && n_panels == 1 && user_K == o.K && user_N == o.N && o.two_layer_tiles >= 0 &&
        (o.K == 32 || o.K == 64 || o.K == 128) && (o.N == 32 || o.N == 64 || o.N == 128))
      build_two_layer_tiles(S, M, Ap, Ai, o.K, o.N, o.compute_units);

    // MultiDimensionalSet-layout view (Fusion_Inspector.h:959-1010).
    const int nt = (int)S->tiles.size();
    std::vector<int> rem_all;
    rem_all.reserve(S->rem_rows.size() + S->long_rows.size());
    for (int i = 0; i < L; ++i)
      if (!fused[i]) rem_all.push_back(i);
    const int nrp = ceil_div((int)rem_all.size(), 64);
    const int P = nt + nrp;
    S->ptr1 = {0, nt, P};
    S->ptr2.assign(P + 1, 0);
    S->ker_begin.assign(2 * (size_t)P, 0);
    S->id.reserve((size_t)M + L);
    S->type.reserve((size_t)M + L);
    S->tile_range.resize(4 * (size_t)nt);
    S->writeback.resize(2 * (size_t)nt);
    for (int p = 0; p < nt; ++p) {
      const auto &t = S->tiles[p];
      for (int r = t.own_begin; r < t.own_end; ++r) { S->id.push_back(r); S->type.push_back(0); }
      S->ker_begin[2 * p] = (int)S->id.size();
      for (int q = t.cons_begin; q < t.cons_end; ++q) { S->id.push_back(S->fused_ids[q]); S->type.push_back(1); }
      S->ker_begin[2 * p + 1] = (int)S->id.size();
      S->ptr2[p + 1] = (int)S->id.size();
      S->tile_range[4 * p + 0] = t.prod_begin; S->tile_range[4 * p + 1] = t.prod_end;
      S->tile_range[4 * p + 2] = t.own_begin;  S->tile_range[4 * p + 3] = t.own_end;
      S->writeback[2 * p] = t.wb_begin; S->writeback[2 * p + 1] = t.wb_end;
    }
    for (int g = 0; g < nrp; ++g) {
      const int p = nt + g;
      S->ker_begin[2 * p] = (int)S->id.size();
      for (int q = g * 64; q < std::min((int)rem_all.size(), (g + 1) * 64); ++q) {
        S->id.push_back(rem_all[q]); S->type.push_back(1);
      }
      S->ker_begin[2 * p + 1] = (int)S->id.size();
      S->ptr2[p + 1] = (int)S->id.size();
    }
    if (gemm_stream) {  // step offsets relative to each tile's first fused id, for the view
      S->view_step_ptr = S->step_ptr;
      for (size_t ti = 0; ti < S->tiles.size(); ++ti) {
        const int st = S->tile_step[ti];
        if (st < 0) continue;
        const int steps = (S->tiles[ti].prod_end - S->tiles[ti].prod_begin + 63) / 64;
        for (int q = 0; q <= steps + 1; ++q) S->view_step_ptr[st + q] -= S->tiles[ti].cons_begin;
      }
    }
  } catch (const std::bad_alloc &) {
    delete S;
    return tf::fail(TF_ENOMEM, "tf_inspect: out of host memory");
  }
  *out = S;
  return TF_OK;
}

extern "C" void tf_schedule_free(tf_schedule *s) {
  if (!s) return;
  tf::release_device_schedule(s->dev);
  delete s;
}

extern "C" tf_status tf_schedule_get_info(const tf_schedule *s, tf_schedule_info *info) {
  if (!s || !info) return tf::fail(TF_EINVAL, "tf_schedule_get_info: null argument");
  tf_schedule_info full;
  std::memset(&full, 0, sizeof(full));
  tf_schedule_info *const caller = info;
  info = &full;
  info->op = s->opts.op; info->N = s->user_N; info->K = s->user_K;
  info->rows = s->L; info->inter_rows = s->M;
  info->n_tiles = (int)s->tiles.size();
  info->n_fused_rows = (int)s->fused_ids.size();
  info->n_remainder_rows = (int)(s->rem_rows.size() + s->zero_rows.size() + s->long_rows.size());
  info->n_long_rows = (int)s->long_rows.size();
  info->n_long_chunks = s->long_part ? (int)s->seg_ptr.size() - 1 : (int)s->long_chunks.size();
  info->long_row_hot_cols = s->long_part ? s->hot_cols : 0;
  info->n_producer_rows = (int)std::min<long long>(s->n_producer_rows, INT_MAX);
  info->n_writeback_rows = s->n_writeback_rows;
  info->max_tile_producer_rows = s->slab_rows;
  info->lds_bytes = s->lds_bytes;
  info->windowed = s->windowed ? 1 : 0;
  info->wide_strips = s->win_wide ? 1 : 0;
  info->streamed = s->gemm_stream ? 1 : 0;
  info->ring_rows = s->ring_rows;
  info->strip_cols = s->windowed ? s->opts.strip_cols : 0;
  info->xcd_chunk_rows = s->xcd_chunk_rows;
  info->fused_nnz = s->fused_nnz;
  info->marched = s->march ? 1 : 0;
  info->march_tile_x = s->march_tile[0];
  info->march_tile_y = s->march_tile[1];
  info->march_slots = s->march_slots;
  info->march_declined = s->march_declined;
  info->register_weights = s->gemm_regw ? 1 : 0;
  info->n_zero_rows = (int)s->zero_rows.size();
  info->two_layer_tiles = (int)s->l2_tiles.size();
  info->intermediate_placed = s->t_pos.empty() ? 0 : 1;
  info->short_row_hot_rows = s->rem_hot_rows;
  {
    long long computed = (long long)s->plain_rows.size();
    for (const auto &t : s->launch_tiles) computed += t.prod_end - t.prod_begin;
    if (s->march) computed = s->n_producer_rows;
    info->n_computed_rows = (int)std::min<long long>(computed, INT_MAX);
  }
  long long ws = 0;
  if (s->march) ws += (long long)s->march_ell_off.size() * 16;  // ELL rows with values, their offsets and sources
  if (s->n_writeback_rows > 0) ws += (long long)s->M * s->opts.N * 4;
  ws += (long long)s->long_chunks.size() * s->opts.N * 4;
  if (s->long_part) ws += ((long long)s->seg_ptr.size() - 1 + (long long)s->seg_groups.size()) * s->opts.N * 4 + (long long)s->seg_src.size() * 4;  // partial sums, regrouped values
  if (s->user_K != s->opts.K) ws += ((long long)s->M + s->opts.N) * s->opts.K * 4;  // padded copies of B and C
  if (s->user_N != s->opts.N) ws += ((long long)s->L + s->opts.K) * s->opts.N * 4;  // one column panel of D and of C
  ws += (long long)s->rem_ptr.size() * 4 + (long long)s->rem_col.size() * 12;       // remainder rows in list order
  info->workspace_bytes = ws;
  return tf::emit_out("tf_schedule_get_info", caller, full, TF_SIZE_THROUGH(tf_schedule_info, march_slots));
}

extern "C" tf_status tf_schedule_get_view(const tf_schedule *s, tf_schedule_view *v) {
  if (!s || !v) return tf::fail(TF_EINVAL, "tf_schedule_get_view: null argument");
  tf_schedule_view full;
  std::memset(&full, 0, sizeof(full));
  tf_schedule_view *const caller = v;
  v = &full;
  v->n1 = 2;
  v->n_part = s->ptr1[2];
  v->n_id = (int)s->id.size();
  v->n_tiles = (int)s->tiles.size();
  v->ptr1 = s->ptr1.data(); v->ptr2 = s->ptr2.data(); v->ker_begin = s->ker_begin.data();
  v->id = s->id.data(); v->type = s->type.data();
  v->tile_range = s->tile_range.data(); v->writeback = s->writeback.data();
  v->tile_step = s->gemm_stream ? s->tile_step.data() : nullptr;
  v->step_ptr = s->gemm_stream ? s->view_step_ptr.data() : nullptr;
  v->n_step_ptr = s->gemm_stream ? (int)s->view_step_ptr.size() : 0;
  v->two_layer_range = s->l2_tiles.empty() ? nullptr : &s->l2_tiles[0].o0;
  v->n_two_layer = (int)s->l2_tiles.size();
  return tf::emit_out("tf_schedule_get_view", caller, full, TF_SIZE_THROUGH(tf_schedule_view, n_step_ptr));
}

extern "C" tf_status tf_schedule_validate(const tf_schedule *s, int L, int M, const int *Ap,
                                          const int *Ai) {
  if (!s || !Ap) return tf::fail(TF_EINVAL, "tf_schedule_validate: null argument");
  if (L != s->L || M != s->M || Ap[L] != s->nnz)
    return tf::fail(TF_ESCHEDULE, "schedule was built for %d x %d with %lld entries, got %d x %d with %d",
                    s->L, s->M, s->nnz, L, M, Ap[L]);
  if (s->march)
    return tf::fail(TF_EINVAL, "tf_schedule_validate: marching runs are checked against both patterns: use tf_schedule_validate_inner");
  const int row_bytes = (s->slab_ld > 0 ? s->slab_ld : s->opts.N) * 4 + (s->gemm_regw ? 16 : 0);
  std::vector<int> owner(M, -1), done(L, 0);
  std::vector<char> stored(M, 0);
  int prev_end = 0;
  for (size_t ti = 0; ti < s->tiles.size(); ++ti) {
    const auto &t = s->tiles[ti];
    if (t.own_begin != prev_end || t.own_end <= t.own_begin)
      return tf::fail(TF_ESCHEDULE, "tile %zu: owned rows [%d,%d) do not continue at %d", ti, t.own_begin, t.own_end, prev_end);
    prev_end = t.own_end;
    if (t.prod_begin > t.own_begin || t.prod_end < t.own_end || t.prod_begin < 0 || t.prod_end > M)
      return tf::fail(TF_ESCHEDULE, "tile %zu: producer range [%d,%d) does not cover owned rows [%d,%d)", ti, t.prod_begin, t.prod_end, t.own_begin, t.own_end);
    if (s->gemm_stream && t.cons_end > t.cons_begin) {
      // rows of step q are computed while rows 64q.. are produced: all their columns were produced
      // in earlier steps and are still among the last ring_rows - 64 rows
      const int st = ti < s->tile_step.size() ? s->tile_step[ti] : -1;
      const int steps = (t.prod_end - t.prod_begin + 63) / 64;
      if (st < 0 || steps > 1024 || st + steps + 2 > (int)s->step_ptr.size() || s->step_ptr[st] != t.cons_begin ||
          s->step_ptr[st + steps + 1] != t.cons_end)
        return tf::fail(TF_ESCHEDULE, "tile %zu: bad step table", ti);
      for (int q = 0; q <= steps; ++q) {
        if (s->step_ptr[st + q + 1] < s->step_ptr[st + q])
          return tf::fail(TF_ESCHEDULE, "tile %zu: step table not monotone at step %d", ti, q);
        if (q < steps && s->step_ptr[st + q + 1] - s->step_ptr[st + q] > s->stream_step_cap)
          return tf::fail(TF_ESCHEDULE, "tile %zu: step %d has more rows than the consumers take", ti, q);
        for (int x = s->step_ptr[st + q]; x < s->step_ptr[st + q + 1]; ++x) {
          const int i = s->fused_ids[x];
          if (i < 0 || i >= L) return tf::fail(TF_ESCHEDULE, "tile %zu: fused row %d out of range", ti, i);
          if (Ap[i + 1] - Ap[i] > s->stream_max_len || Ap[i + 1] == Ap[i])
            return tf::fail(TF_ESCHEDULE, "tile %zu: fused row %d has %d entries", ti, i, Ap[i + 1] - Ap[i]);
          if (s->fused_rec[4 * (size_t)x] != i || s->fused_rec[4 * (size_t)x + 1] != Ap[i] || s->fused_rec[4 * (size_t)x + 2] != Ap[i + 1])
            return tf::fail(TF_ESCHEDULE, "tile %zu: record of fused row %d does not match the matrix", ti, i);
          for (int k = Ap[i]; k < Ap[i + 1]; ++k) {
            if (Ai[k] < t.prod_begin || Ai[k] >= t.prod_end) continue;  // reported below
            const int qc = (Ai[k] - t.prod_begin) / 64;
            if (qc > q - 1 || qc < q - s->ring_rows / 64 + 1)
              return tf::fail(TF_ESCHEDULE, "fused row %d in step %d of tile %zu reads intermediate row %d that is not in the ring then", i, q, ti, Ai[k]);
          }
        }
      }
    }
    if (!s->windowed && !s->gemm_stream && t.cons_end > t.cons_begin &&
        (long long)(t.prod_end - t.prod_begin) * row_bytes > s->opts.lds_budget_bytes)
      return tf::fail(TF_ESCHEDULE, "tile %zu: slab of %d rows exceeds the LDS budget", ti, t.prod_end - t.prod_begin);
    if (t.wb_begin < t.own_begin || t.wb_end > t.own_end || t.wb_end < t.wb_begin)
      return tf::fail(TF_ESCHEDULE, "tile %zu: write-back range [%d,%d) outside owned rows", ti, t.wb_begin, t.wb_end);
    for (int r = t.own_begin; r < t.own_end; ++r) owner[r] = (int)ti;
    for (int r = t.wb_begin; r < t.wb_end; ++r) stored[r] = 1;
    if (t.cons_begin < 0 || t.cons_end > (int)s->fused_ids.size() || t.cons_end < t.cons_begin)
      return tf::fail(TF_ESCHEDULE, "tile %zu: bad fused id range", ti);
    for (int q = t.cons_begin; q < t.cons_end; ++q) {
      const int i = s->fused_ids[q];
      if (i < 0 || i >= L) return tf::fail(TF_ESCHEDULE, "tile %zu: fused row %d out of range", ti, i);
      if (done[i]++) return tf::fail(TF_ESCHEDULE, "second-op row %d scheduled twice", i);
      for (int k = Ap[i]; k < Ap[i + 1]; ++k)
        if (Ai[k] < t.prod_begin || Ai[k] >= t.prod_end)
          return tf::fail(TF_ESCHEDULE, "fused row %d reads intermediate row %d outside tile %zu [%d,%d)", i, Ai[k], ti, t.prod_begin, t.prod_end);
    }
  }
  if (prev_end != M) return tf::fail(TF_ESCHEDULE, "owned rows end at %d, expected %d", prev_end, M);
  auto check_rem = [&](int i) -> tf_status {
    if (i < 0 || i >= L) return tf::fail(TF_ESCHEDULE, "remainder row %d out of range", i);
    for (int k = Ap[i]; k < Ap[i + 1]; ++k)
      if (!stored[Ai[k]])
        return tf::fail(TF_ESCHEDULE, "remainder row %d reads intermediate row %d that no tile stores", i, Ai[k]);
    return TF_OK;
  };
  // Where a row of the intermediate is stored: its own index, or its place in the list of rows the GEMM computes.
  if (!s->t_pos.empty()) {
    if ((int)s->t_pos.size() != M || !s->launch_tiles.empty() || !s->long_chunks.empty() || (!s->rem_rows.empty() && s->rem_ptr.empty()))
      return tf::fail(TF_ESCHEDULE, "placed intermediate: a consumer would read rows at their own index");
    std::vector<int> count(M, 0);
    for (size_t q = 0; q < s->plain_rows.size(); ++q) {
      const int r = s->plain_rows[q];
      if (r < 0 || r >= M || s->t_pos[r] != (int)q) return tf::fail(TF_ESCHEDULE, "placed intermediate: row %d is not where the list puts it", r);
      ++count[r];
    }
    for (int r = 0; r < M; ++r)
      if ((count[r] == 0) != (s->t_pos[r] < 0) || count[r] > 1) return tf::fail(TF_ESCHEDULE, "placed intermediate: row %d has no single place", r);
  }
  auto tcol = [&](int c) { return s->t_pos.empty() ? c : s->t_pos[c]; };
  if (!s->rem_ptr.empty()) {  // the rows of the list stored in list order must be A's rows, entry for entry
    if (s->rem_ptr.size() != s->rem_rows.size() + 1 || s->rem_ptr[0] != 0 || s->rem_ptr.back() != (int)s->rem_col.size() || s->rem_src.size() != s->rem_col.size())
      return tf::fail(TF_ESCHEDULE, "remainder rows in list order: bad tables");
    for (size_t q = 0; q < s->rem_rows.size(); ++q) {
      const int i = s->rem_rows[q];
      if (i < 0 || i >= L || s->rem_ptr[q + 1] - s->rem_ptr[q] != Ap[i + 1] - Ap[i])
        return tf::fail(TF_ESCHEDULE, "remainder rows in list order: row %d has another length than in A", i);
      for (int k = Ap[i], e = s->rem_ptr[q]; k < Ap[i + 1]; ++k, ++e)
        if (s->rem_src[e] != k || (s->rem_col[e] & INT_MAX) != tcol(Ai[k])) return tf::fail(TF_ESCHEDULE, "remainder rows in list order: row %d differs from A's", i);
    }
  }
  for (int i : s->zero_rows) {
    if (i < 0 || i >= L) return tf::fail(TF_ESCHEDULE, "empty row %d out of range", i);
    if (done[i]++) return tf::fail(TF_ESCHEDULE, "second-op row %d scheduled twice", i);
    if (Ap[i + 1] != Ap[i]) return tf::fail(TF_ESCHEDULE, "row %d is listed as empty and has entries", i);
  }
  for (int i : s->rem_rows) {
    if (i < 0 || i >= L) return tf::fail(TF_ESCHEDULE, "remainder row %d out of range", i);
    if (done[i]++) return tf::fail(TF_ESCHEDULE, "second-op row %d scheduled twice", i);
    if (Ap[i + 1] - Ap[i] > s->opts.long_row_nnz)
      return tf::fail(TF_ESCHEDULE, "remainder row %d is long but not chunked", i);
    if (tf_status rc = check_rem(i)) return rc;
  }
  if (s->long_part) {
    const int n_seg = (int)s->seg_ptr.size() - 1, n_hot_seg = 8 * s->seg_per_xcd;
    if (n_seg < n_hot_seg || s->seg_ptr.empty() || s->seg_ptr[0] != 0 || s->seg_ptr[n_seg] != (int)s->seg_src.size() ||
        s->seg_col.size() != s->seg_src.size())
      return tf::fail(TF_ESCHEDULE, "long-row segments: bad tables");
    std::vector<signed char> reader(M, -1);  // partition through which an intermediate row is read
    std::vector<char> seen(s->nnz > 0 ? (size_t)s->nnz : 1, 0);
    std::vector<char> seg_used(n_seg, 0);
    for (const auto &lr : s->long_rows) {
      if (tf_status rc = check_rem(lr.row)) return rc;
      if (done[lr.row]++) return tf::fail(TF_ESCHEDULE, "second-op row %d scheduled twice", lr.row);
      if (lr.first < 0 || lr.count < 0 || lr.first + lr.count > (int)s->lrow_seg.size())
        return tf::fail(TF_ESCHEDULE, "long row %d: bad segment range", lr.row);
      long long covered = 0;
      std::vector<int> segs;  // the row's segments, groups expanded
      for (int q = lr.first; q < lr.first + lr.count; ++q) {
        const int slot = s->lrow_seg[q];
        if (slot >= n_seg) {
          if (slot - n_seg >= (int)s->seg_groups.size()) return tf::fail(TF_ESCHEDULE, "long row %d: unknown group slot %d", lr.row, slot);
          const auto &g = s->seg_groups[slot - n_seg];
          if (g.row != slot || g.count <= 0 || g.count > 32 || g.first < 0 || g.first + g.count > (int)s->lrow_seg.size())
            return tf::fail(TF_ESCHEDULE, "long row %d: bad group %d", lr.row, slot - n_seg);
          segs.insert(segs.end(), s->lrow_seg.begin() + g.first, s->lrow_seg.begin() + g.first + g.count);
        } else {
          segs.push_back(slot);
        }
      }
      for (const int sg : segs) {
        if (sg < 0 || sg >= n_seg || seg_used[sg]++) return tf::fail(TF_ESCHEDULE, "long row %d: segment %d unknown or used twice", lr.row, sg);
        const int cls = sg < n_hot_seg ? sg / s->seg_per_xcd : -2;
        if (s->seg_ptr[sg + 1] - s->seg_ptr[sg] > 64 || s->seg_ptr[sg + 1] <= s->seg_ptr[sg])
          return tf::fail(TF_ESCHEDULE, "long row %d: segment %d is empty or longer than 64", lr.row, sg);
        int prev = -1;
        for (int e = s->seg_ptr[sg]; e < s->seg_ptr[sg + 1]; ++e) {
          const int k = s->seg_src[e];
          if (k < Ap[lr.row] || k >= Ap[lr.row + 1] || seen[k]++ || k <= prev || (s->seg_col[e] & INT_MAX) != tcol(Ai[k]))
            return tf::fail(TF_ESCHEDULE, "long row %d: segment %d does not hold entries of the row once, in order", lr.row, sg);
          prev = k;
          if (cls >= 0) {  // (cold segments may read any row)
            signed char &ow = reader[Ai[k]];
            if (ow == -1) ow = (signed char)cls;
            else if (ow != cls) return tf::fail(TF_ESCHEDULE, "intermediate row %d is read through two partitions", Ai[k]);
          }
          ++covered;
        }
      }
      if (covered != Ap[lr.row + 1] - Ap[lr.row]) return tf::fail(TF_ESCHEDULE, "long row %d: segments hold %lld of its %d entries", lr.row, covered, Ap[lr.row + 1] - Ap[lr.row]);
    }
    for (int sg = 0; sg < n_seg; ++sg)
      if (!seg_used[sg] && s->seg_ptr[sg + 1] != s->seg_ptr[sg]) return tf::fail(TF_ESCHEDULE, "segment %d belongs to no row", sg);
  }
  for (const auto &lr : s->long_rows) {
    if (s->long_part) break;
    if (tf_status rc = check_rem(lr.row)) return rc;
    if (done[lr.row]++) return tf::fail(TF_ESCHEDULE, "second-op row %d scheduled twice", lr.row);
    int k = Ap[lr.row];
    if (lr.first < 0 || lr.count <= 0 || lr.first + lr.count > (int)s->long_chunks.size())
      return tf::fail(TF_ESCHEDULE, "long row %d: bad chunk range", lr.row);
    for (int c = lr.first; c < lr.first + lr.count; ++c) {
      const auto &ch = s->long_chunks[c];
      if (ch.row != lr.row || ch.k_begin != k || ch.k_end <= ch.k_begin || ch.slot != c ||
          ch.k_end - ch.k_begin > std::max(s->opts.long_row_nnz, 1024))
        return tf::fail(TF_ESCHEDULE, "long row %d: chunk %d does not continue at entry %d", lr.row, c, k);
      k = ch.k_end;
    }
    if (k != Ap[lr.row + 1]) return tf::fail(TF_ESCHEDULE, "long row %d: chunks end at %d, row ends at %d", lr.row, k, Ap[lr.row + 1]);
  }
  for (int i = 0; i < L; ++i)
    if (done[i] != 1) return tf::fail(TF_ESCHEDULE, "second-op row %d scheduled %d times", i, done[i]);
  // Two-layer tiles: the owned ranges partition the rows in order; every owned row reads only hidden rows of its
  // tile, every hidden row of a tile only rows of the first intermediate that the tile computes; both slabs fit.
  if (!s->l2_tiles.empty()) {
    const int H = s->opts.K, N2 = s->opts.N;
    if (L != M) return tf::fail(TF_ESCHEDULE, "two-layer tiles on a matrix that is not square");
    if (s->l2_lds_bytes > kMaxLds) return tf::fail(TF_ESCHEDULE, "two-layer tiles: %d bytes of LDS", s->l2_lds_bytes);
    int end = 0;
    for (size_t ti = 0; ti < s->l2_tiles.size(); ++ti) {
      const tf::Tile2 &t = s->l2_tiles[ti];
      if (t.o0 != end || t.o1 <= t.o0 || t.o1 > L) return tf::fail(TF_ESCHEDULE, "two-layer tile %zu owns [%d, %d) after row %d", ti, t.o0, t.o1, end);
      end = t.o1;
      if (t.h0 < 0 || t.h1 < t.h0 || t.h1 > M || t.t0 < 0 || t.t1 < t.t0 || t.t1 > M)
        return tf::fail(TF_ESCHEDULE, "two-layer tile %zu: bad ranges", ti);
      const long long PH = t.h1 - t.h0, P1 = t.t1 - t.t0, b_floats = t.c_off - t.b_off;
      const int c0 = PH > 0 ? std::min(t.o0, t.h0) : t.o0, c1 = PH > 0 ? std::max(t.o1, t.h1) : t.o1;
      const long long c_floats = ((c1 - c0 + 1 + 3) / 4 * 4) + 2LL * ((Ap[c1] - Ap[c0] + 3) / 4 * 4);
      if (t.b_off < 0 || (t.b_off & 3) || (t.c_off & 3) || P1 * (H + tf::kTile2Pad) > t.b_off || PH * (N2 + tf::kTile2Pad) > t.b_off ||
          PH * (H + tf::kTile2Pad) > b_floats || tf::kTile2StageFloats > b_floats || (t.c_off + c_floats) * 4 > s->l2_lds_bytes)
        return tf::fail(TF_ESCHEDULE, "two-layer tile %zu: %lld hidden and %lld intermediate rows and its %d entries of A do not fit LDS", ti, PH, P1, Ap[c1] - Ap[c0]);
      for (int i = t.o0; i < t.o1; ++i)
        for (int k = Ap[i]; k < Ap[i + 1]; ++k)
          if (Ai[k] < t.h0 || Ai[k] >= t.h1) return tf::fail(TF_ESCHEDULE, "two-layer tile %zu: row %d reads hidden row %d outside [%d, %d)", ti, i, Ai[k], t.h0, t.h1);
      for (int j = t.h0; j < t.h1; ++j)
        for (int k = Ap[j]; k < Ap[j + 1]; ++k)
          if (Ai[k] < t.t0 || Ai[k] >= t.t1) return tf::fail(TF_ESCHEDULE, "two-layer tile %zu: hidden row %d reads row %d outside [%d, %d)", ti, j, Ai[k], t.t0, t.t1);
    }
    if (end != L) return tf::fail(TF_ESCHEDULE, "two-layer tiles end at row %d of %d", end, L);
  }
  return TF_OK;
}

// The same check, plus what only the inner pattern can show: that a windowed tile's window of C
// holds every row its producer rows read, and that window, slab and tables fit the tile's LDS.
extern "C" tf_status tf_schedule_validate_inner(const tf_schedule *s, int L, int M, const int *Ap, const int *Ai,
                                                const int *inner_Ap, const int *inner_Ai, int inner_cols) {
  if (s && s->march) {
    if (!Ap || !inner_Ap || L != s->L || M != s->M || L != M || Ap[L] != s->nnz)
      return tf::fail(TF_ESCHEDULE, "tf_schedule_validate_inner: the schedule's runs were built for other patterns");
    if (inner_cols != s->opts.inner_cols || inner_Ap[M] != s->inner_nnz || tf_pattern_hash(M, inner_Ap, inner_Ai) != s->inner_hash ||
        tf_pattern_hash(L, Ap, Ai) != s->pattern_hash)
      return tf::fail(TF_ESCHEDULE, "the schedule's runs were built from another inner pattern");
    return tf::validate_march(s, M, Ap, Ai, inner_Ap, inner_Ai);
  }
  if (tf_status rc = tf_schedule_validate(s, L, M, Ap, Ai)) return rc;
  if (!s->windowed) return TF_OK;
  if (!inner_Ap || (!inner_Ai && inner_Ap[M] > 0))
    return tf::fail(TF_EINVAL, "tf_schedule_validate_inner: the schedule has windowed tiles; the inner pattern is needed");
  if (inner_cols != s->opts.inner_cols || inner_Ap[M] != s->inner_nnz || tf_pattern_hash(M, inner_Ap, inner_Ai) != s->inner_hash)
    return tf::fail(TF_ESCHEDULE, "the schedule's windows were built from another inner pattern");
  if (s->win.size() != 2 * s->tiles.size()) return tf::fail(TF_ESCHEDULE, "windowed schedule: %zu windows for %zu tiles", s->win.size() / 2, s->tiles.size());
  auto a16 = [](long long x) { return (x + 15) / 16 * 16; };
  const int SW = s->opts.strip_cols;
  for (size_t ti = 0; ti < s->tiles.size(); ++ti) {
    const auto &t = s->tiles[ti];
    const int w0 = s->win[2 * ti], w1 = s->win[2 * ti + 1];
    if (w0 < 0 || w1 < w0 || w1 > inner_cols) return tf::fail(TF_ESCHEDULE, "tile %zu: bad window [%d,%d)", ti, w0, w1);
    for (int r = t.prod_begin; r < t.prod_end; ++r)
      for (int k = inner_Ap[r]; k < inner_Ap[r + 1]; ++k)
        if (inner_Ai[k] < w0 || inner_Ai[k] >= w1)
          return tf::fail(TF_ESCHEDULE, "tile %zu: producer row %d reads row %d of C outside the window [%d,%d)", ti, r, inner_Ai[k], w0, w1);
    const long long P = t.prod_end - t.prod_begin, R = t.own_end - t.own_begin, nz = (long long)inner_Ap[t.prod_end] - inner_Ap[t.prod_begin];
    const long long lds = s->win_wide ? a16(4 * (P + 1)) + a16(4 * (R + 1)) + 4LL * SW * (w1 - w0 + P)
                                      : a16(4 * (P + 1)) + a16(4 * R) + a16(8 * (nz + 2 * P)) + 4LL * SW * (w1 - w0 + P);
    if (lds > s->lds_bytes || lds > kMaxLds)
      return tf::fail(TF_ESCHEDULE, "tile %zu: window, slab and tables take %lld bytes of LDS, the kernel is launched with %d", ti, lds, s->lds_bytes);
  }
  return TF_OK;
}
