// Marching runs: the fused SpMM-SpMM schedule for stencil-like patterns.
//
// On a three-dimensional grid no contiguous range of rows holds a row's dependences (the
// neighbours in the next plane are nx*ny rows away), so tiles of consecutive rows fuse
// nothing.  The reference's answer is tiling with redundancy: a tile recomputes the halo
// rows of the intermediate it needs (fusion/src/SpMM_SpMM.cpp:984-1057,
// fusion/src/SparseFusionWithRedundancy.cpp:11-33).  Here a tile is a *run*: a column of
// grid points (bx x by per plane) that one workgroup walks plane by plane, keeping in LDS
// only the rows of C and of the intermediate that the next planes still need.  Halo rows
// of the intermediate (the ring around the column) are recomputed by the run; rows of C are
// fetched from memory once per run that needs them.
//
// The grid only says how rows are dealt to runs and steps.  Which rows a run has to load,
// recompute and keep, and for how long, is derived from the two sparsity patterns alone,
// and tf_schedule_validate replays every run against them -- so a wrong grid hint can make a
// schedule slow or impossible, never wrong.
#include <algorithm>
#include <climits>
#include <cstring>
#include <iterator>
#include <map>
#include <vector>

#include "tf_internal.h"

namespace tf {

namespace {

constexpr int kMaxLds = 163840;

// The grid a pattern was generated on, from the distances between a row and its columns: a
// 7-point-like stencil on nx x ny x nz points, x fastest, has the distances 1, nx and nx*ny; a
// 5-point-like stencil on nx x n points the distances 1 and nx (a grid of nx x 1 x n: the runs then
// walk the grid's lines, a stretch of a line at a time).  Stencils with diagonal neighbours (9, 19, 27
// points) have the distances |a + b nx + c nx ny| with a, b, c in -1 .. 1: up to thirteen of them.
bool detect_grid(int M, const int *Ap, const int *Ai, int grid[3]) {
  std::map<int, long long> dist;
  for (int i = 0; i < M; ++i)
    for (int k = Ap[i]; k < Ap[i + 1]; ++k) {
      const int d = std::abs(Ai[k] - i);
      if (d == 0) continue;
      if (dist.size() >= 13 && !dist.count(d)) return false;
      ++dist[d];
    }
  if (dist.size() == 2) {
    const int d1 = dist.begin()->first, d2 = std::next(dist.begin())->first;
    if (d1 == 1 && d2 >= 16 && M % d2 == 0 && M / d2 >= 2) {
      grid[0] = d2; grid[1] = 1; grid[2] = M / d2;
      return true;
    }
  }
  if (dist.size() == 3) {
    auto it = dist.begin();
    const int d1 = it->first; ++it;
    const int d2 = it->first; ++it;
    const int d3 = it->first;
    if (d1 == 1 && d2 >= 2 && d3 % d2 == 0 && d3 / d2 >= 2 && M % d3 == 0 && M / d3 >= 2) {
      grid[0] = d2; grid[1] = d3 / d2; grid[2] = M / d3;
      return true;
    }
  }
  // diagonal neighbours: the second distance is nx - 1 or nx, the first one beyond nx + 1 one of the plane's
  if (dist.size() < 2 || dist.begin()->first != 1) return false;
  std::vector<int> D;
  for (const auto &kv : dist) D.push_back(kv.first);
  auto all_fit = [&](long long nx, long long P) {
    for (int d : D) {
      bool ok = false;
      for (int c = -1; c <= 1 && !ok; ++c)
        for (int b = -1; b <= 1 && !ok; ++b)
          for (int a = -1; a <= 1 && !ok; ++a) ok = std::llabs(a + b * nx + c * P) == d;
      if (!ok) return false;
    }
    return true;
  };
  for (const int nx : {D[1], D[1] + 1}) {
    if (nx < 3 || M % nx != 0) continue;
    auto far = std::upper_bound(D.begin(), D.end(), nx + 1);
    if (far == D.end()) {  // a flat grid
      if (nx >= 16 && M / nx >= 2 && all_fit(nx, (long long)M * 4)) {
        grid[0] = nx; grid[1] = 1; grid[2] = M / nx;
        return true;
      }
      continue;
    }
    for (const int P : {*far + nx + 1, *far + nx, *far + nx - 1, *far + 1, *far, *far - 1})
      if (P > 0 && P % nx == 0 && P / nx >= 2 && M % P == 0 && M / P >= 2 && all_fit(nx, P)) {
        grid[0] = nx; grid[1] = P / nx; grid[2] = M / P;
        return true;
      }
  }
  return false;
}

}  // namespace

bool build_march(tf_schedule *S, int M, const int *Ap, const int *Ai, const int *Bp, const int *Bi,
                 const tf_inspect_opts &o, const tf_inspect_opts &given) {
  // (every way out says why in S->march_declined, which tf_schedule_get_info reports)
  auto decline = [&](int why) { S->march_declined = why; return false; };
  if (S->L != M || o.inner_cols != M || o.N % 64 != 0) return decline(TF_MARCH_SHAPE);
  const long long nnzA = Ap[M], nnzB = Bp[M];
  if (nnzA >= kMarchSrcA || nnzB >= kMarchSrcA) return decline(TF_MARCH_SHAPE);
  // the kernel reaches the rows of C and its lists through 32-bit byte offsets (row * 4N by a 24-bit multiply)
  if (M >= (1 << 24) || (long long)M * o.N * 4 >= (1LL << 32)) return decline(TF_MARCH_SHAPE);
  int width = 0;
  for (int i = 0; i < M; ++i) {
    if (Ap[i + 1] - Ap[i] > kMarchWideW || Bp[i + 1] - Bp[i] > kMarchWideW) return decline(TF_MARCH_ROW_TOO_LONG);
    width = std::max(width, std::max(Ap[i + 1] - Ap[i], Bp[i + 1] - Bp[i]));
  }
  int grid[3] = {given.grid_nx, given.grid_ny, given.grid_nz};
  if (grid[0] > 0 || grid[1] > 0 || grid[2] > 0) {
    if (grid[0] <= 0 || grid[1] <= 0 || grid[2] <= 0 || (long long)grid[0] * grid[1] * grid[2] != M) return decline(TF_MARCH_NO_GRID);
  } else if (!detect_grid(M, Ap, Ai, grid)) {
    return decline(TF_MARCH_NO_GRID);
  }
  const int nx = grid[0], ny = grid[1], nz = grid[2];
  const int ell_w = march_ell_stride(width);  // pairs per ELL row: 8, or 32 when a row has more than 8 entries
  const int slot_budget = (kMaxLds - kMarchSlot0) / kMarchRowBytes;

  // Runs: columns of bx x by points, cut along z so that every compute unit gets a run.
  auto attempt = [&](int bx, int by) -> bool {
    const int tx = (nx + bx - 1) / bx, ty = (ny + by - 1) / by;
    const int per_plane = tx * ty;
    int nzc = std::max(1, (o.compute_units + per_plane - 1) / per_plane);
    nzc = std::min(nzc, std::max(1, nz / 8));  // a run of a few planes is mostly start-up
    // (a run's table of iterations has kMarchMaxIter places: taller grids are cut further, into a whole
    // number of turns of the compute units where that is near)
    const int nzc_min = (nz + kMarchMaxIter - 9) / (kMarchMaxIter - 8);
    if (nzc < nzc_min) {
      nzc = nzc_min;
      for (int c = nzc_min; c <= 2 * nzc_min; ++c)
        if ((long long)per_plane * c % o.compute_units == 0) { nzc = c; break; }
    }
    // When the runs are more than the compute units but not a whole number of turns of them (352 columns on 256
    // units: the second turn is a third full), more cuts along z fill the last turn -- against the three or so
    // iterations of start-up that every run pays: the number of cuts with the best product of the two.
    if (per_plane * nzc > o.compute_units) {
      auto score = [&](int c) {
        const long long n = (long long)per_plane * c, turns = (n + o.compute_units - 1) / o.compute_units;
        const double len = (double)nz / c;
        return (double)n / (double)(turns * o.compute_units) * len / (len + 3.0);
      };
      int best = nzc;
      for (int c = nzc + 1; c <= std::min(std::max(1, nz / 8), 8 * nzc); ++c)
        if (score(c) > score(best) + 0.02) best = c;
      nzc = best;
    }
    const int zlen = (nz + nzc - 1) / nzc;

    std::vector<int> runs, row_ptr, load_ptr, load, row_out, row_id, ell_off, ell_src, ids;
    std::vector<TileDesc> tiles;
    std::vector<int> firstT(M), lastT(M), stampT(M, -1), slotT(M), firstC(M), lastC(M), stampC(M, -1), slotC(M);
    std::vector<std::vector<int>> dstep, tgroup, cgroup, rel;
    std::vector<int> free_slots;
    int max_slots = 0, max_t = 0, max_d = 0, max_loads = 0;
    long long produced = 0;
    // row_ptr holds two entries per iteration (its intermediate rows begin at [2i], its second-op
    // rows at [2i+1]) and one more at the very end; load_ptr one per iteration and one more
    row_ptr.push_back(0);
    load_ptr.push_back(0);
    int run = 0;
    for (int zc = 0; zc < nzc; ++zc) {
      const int z0 = zc * zlen, z1 = std::min(nz, z0 + zlen);
      if (z0 >= z1) break;
      for (int tyi = 0; tyi < ty; ++tyi)
        for (int txi = 0; txi < tx; ++txi, ++run) {
          const int steps = z1 - z0;
          dstep.assign(steps, {});
          tgroup.assign(steps, {});
          for (int s = 0; s < steps; ++s)
            for (int y = tyi * by; y < std::min(ny, (tyi + 1) * by); ++y)
              for (int x = txi * bx; x < std::min(nx, (txi + 1) * bx); ++x)
                dstep[s].push_back(((z0 + s) * ny + y) * nx + x);
          // intermediate rows by the step that first reads them, and their last reader
          for (int s = 0; s < steps; ++s)
            for (int i : dstep[s])
              for (int k = Ap[i]; k < Ap[i + 1]; ++k) {
                const int t = Ai[k];
                if (stampT[t] != run) { stampT[t] = run; firstT[t] = s; tgroup[s].push_back(t); }
                lastT[t] = s;
              }
          // The first step needs every intermediate row around it at once (three planes of a stencil),
          // later steps one more plane each.  So that every iteration has about the same work, the first
          // group is spread over warm-up iterations that come before the first step and have no
          // second-op rows: an iteration takes as many rows as the largest later group, rounded up to
          // whole rounds of the lane groups.
          size_t steady_t = 1;
          for (int s = 1; s < steps; ++s) steady_t = std::max(steady_t, tgroup[s].size());
          const size_t cap_t = kMarchGroups * std::min<size_t>(kMarchTpg, (steady_t + kMarchGroups - 1) / kMarchGroups);
          const int warm = tgroup[0].size() > cap_t ? (int)((tgroup[0].size() + cap_t - 1) / cap_t) - 1 : 0;
          const int n_iter = steps + warm;
          if (n_iter > kMarchMaxIter) return false;
          if (warm > 0) {
            std::sort(tgroup[0].begin(), tgroup[0].end());
            std::vector<std::vector<int>> tg(n_iter), ds(n_iter);
            const size_t first_len = tgroup[0].size() - (size_t)warm * cap_t;  // the earliest iteration takes the odd part
            size_t pos = 0;
            for (int w = 0; w <= warm; ++w) {
              const size_t len = w == 0 ? first_len : cap_t;
              tg[w].assign(tgroup[0].begin() + pos, tgroup[0].begin() + pos + len);
              pos += len;
            }
            for (int s = 1; s < steps; ++s) tg[warm + s].swap(tgroup[s]);
            for (int s = 0; s < steps; ++s) ds[warm + s].swap(dstep[s]);
            tgroup.swap(tg);
            dstep.swap(ds);
            for (int g = 0; g < n_iter; ++g)
              for (int t : tgroup[g]) lastT[t] += warm;
          }
          // rows of C by the group of intermediate rows that first reads them
          cgroup.assign(n_iter, {});
          for (int g = 0; g < n_iter; ++g) {
            std::sort(tgroup[g].begin(), tgroup[g].end());
            for (int t : tgroup[g])
              for (int k = Bp[t]; k < Bp[t + 1]; ++k) {
                const int c = Bi[k];
                if (stampC[c] != run) { stampC[c] = run; firstC[c] = g; cgroup[g].push_back(c); }
                lastC[c] = g;
              }
          }
          // ... and the same levelling for the rows of C: what a list holds beyond the lane groups' rounds
          // is fetched an iteration earlier (the list before the first iteration takes any number)
          {
            size_t steady_c = 1;
            for (int g = warm + 2; g < n_iter; ++g) steady_c = std::max(steady_c, cgroup[g].size());
            const size_t cap_c = kMarchGroups * std::min<size_t>(kMarchLpg, (steady_c + kMarchGroups - 1) / kMarchGroups);
            for (int g = n_iter - 1; g >= 1; --g) {
              std::sort(cgroup[g].begin(), cgroup[g].end());
              while (cgroup[g].size() > cap_c) { cgroup[g - 1].push_back(cgroup[g].back()); cgroup[g].pop_back(); }
            }
          }
          // Slots, in half iterations: iteration i is phase 2i (the intermediate rows of group i, read from
          // slots of C, written to their slots) and phase 2i+1 (the second-op rows of step i, read from
          // slots of the intermediate, while the rows of C of group i+1 are written to theirs).  A row of
          // C of group g..l is written in phase 2g-1 and last read in phase 2l; an intermediate row first
          // read by step f and last by step l is written in phase 2f and last read in phase 2l+1.  A slot
          // takes a new row only in a phase after its last read.
          rel.assign(2 * n_iter + 4, {});  // rel[p + 1]: slots free from phase p on
          free_slots.clear();
          int next_slot = 0;
          auto take = [&]() {
            if (!free_slots.empty()) { const int s = free_slots.back(); free_slots.pop_back(); return s; }
            return next_slot++;
          };
          runs.push_back((int)row_ptr.size() / 2);
          runs.push_back(n_iter);
          TileDesc td{};
          td.cons_begin = (int)ids.size();
          int lo = INT_MAX, hi = -1;
          for (int ph = -1; ph < 2 * n_iter; ++ph) {
            for (int s : rel[ph + 1]) free_slots.push_back(s);
            if (ph & 1) {  // phase 2g-1: the rows of C of group g arrive
              const int g = (ph + 1) / 2;
              if (g < n_iter) {
                std::sort(cgroup[g].begin(), cgroup[g].end());
                for (int c : cgroup[g]) {
                  slotC[c] = take();
                  rel[2 * lastC[c] + 1 + 1].push_back(slotC[c]);
                  load.push_back(c);
                  load.push_back(kMarchSlot0 + slotC[c] * kMarchRowBytes);
                }
                load_ptr.push_back((int)load.size() / 2);
                if (g > 0) max_loads = std::max(max_loads, (int)cgroup[g].size());
              }
              if (ph >= 1) {  // ... beside the second-op rows of step g-1
                for (int i : dstep[g - 1]) {
                  row_out.push_back(i);
                  row_id.push_back(i);
                  ids.push_back(i);
                  lo = std::min(lo, i); hi = std::max(hi, i);
                  for (int k = Ap[i]; k < Ap[i] + ell_w; ++k) {
                    const bool real = k < Ap[i + 1];
                    ell_off.push_back(real ? kMarchSlot0 + slotT[Ai[k]] * kMarchRowBytes : kMarchZeroOff);
                    ell_src.push_back(real ? (k | kMarchSrcA) : -1);
                  }
                }
                row_ptr.push_back((int)row_out.size());
                max_d = std::max(max_d, (int)dstep[g - 1].size());
              }
            } else {  // phase 2i: the intermediate rows of group i
              const int it = ph / 2;
              for (int t : tgroup[it]) {
                slotT[t] = take();
                rel[2 * lastT[t] + 1 + 1 + 1].push_back(slotT[t]);
                row_out.push_back(~(kMarchSlot0 + slotT[t] * kMarchRowBytes));
                row_id.push_back(t);
                for (int k = Bp[t]; k < Bp[t] + ell_w; ++k) {
                  const bool real = k < Bp[t + 1];
                  ell_off.push_back(real ? kMarchSlot0 + slotC[Bi[k]] * kMarchRowBytes : kMarchZeroOff);
                  ell_src.push_back(real ? k : -1);
                }
              }
              row_ptr.push_back((int)row_out.size());
              produced += (long long)tgroup[it].size();
              max_t = std::max(max_t, (int)tgroup[it].size());
            }
            if (next_slot > slot_budget) return false;
          }
          max_slots = std::max(max_slots, next_slot);
          td.cons_end = (int)ids.size();
          td.own_begin = td.prod_begin = td.wb_begin = td.wb_end = lo == INT_MAX ? 0 : lo;
          td.own_end = td.prod_end = hi + 1;
          tiles.push_back(td);
        }
    }
    // (the kernel reaches its lists through 32-bit byte offsets: 8 bytes per pair of an ELL row and per load-list entry)
    if ((long long)row_out.size() * ell_w * 8 >= (1LL << 32) || (long long)load.size() * 4 >= (1LL << 32) ||
        max_t > kMarchTpg * kMarchGroups || max_d > kMarchDpg * kMarchGroups ||
        max_loads > kMarchLpg * kMarchGroups || (int)ids.size() != M)
      return false;
    S->march = true;
    S->march_grid[0] = nx; S->march_grid[1] = ny; S->march_grid[2] = nz;
    S->march_tile[0] = bx; S->march_tile[1] = by;
    S->march_slots = max_slots;
    S->march_width = width;
    S->march_tpg = std::max(1, (max_t + kMarchGroups - 1) / kMarchGroups);
    S->march_dpg = std::max(1, (max_d + kMarchGroups - 1) / kMarchGroups);
    S->march_lpg = std::max(1, (max_loads + kMarchGroups - 1) / kMarchGroups);
    S->march_runs.swap(runs);
    S->march_row_ptr.swap(row_ptr);
    S->march_load_ptr.swap(load_ptr);
    S->march_load.swap(load);
    S->march_row_out.swap(row_out);
    S->march_row_id.swap(row_id);
    S->march_ell_off.swap(ell_off);
    S->march_ell_src.swap(ell_src);
    S->tiles.swap(tiles);
    S->launch_tiles = S->tiles;
    S->fused_ids.swap(ids);
    S->n_producer_rows = produced;
    S->slab_rows = max_slots;
    S->lds_bytes = kMarchSlot0 + max_slots * kMarchRowBytes;
    S->fused_nnz = nnzA;
    S->inner_nnz = nnzB;
    S->inner_hash = (Bp == Ap && Bi == Ai) ? S->pattern_hash : tf_pattern_hash(M, Bp, Bi);
    return true;
  };

  bool ok = false;
  if (given.march_tile_x > 0 && given.march_tile_y > 0) {
    ok = attempt(given.march_tile_x, given.march_tile_y);
  } else {
    // the largest column that fits: the halo ring costs less the larger the column is
    if (ny >= 8) {
      const int cand[][2] = {{8, 8}, {8, 7}, {8, 6}, {8, 5}, {8, 4}, {4, 4}};
      for (const auto &c : cand)
        if ((ok = attempt(c[0], c[1]))) break;
    } else {  // a flat grid: the column takes all of y and as much of x as gives it the same number of points
      for (const int points : {64, 56, 48, 40, 32, 16}) {
        const int bx = std::min(nx, points / ny);
        if (bx >= 1 && (ok = attempt(bx, ny))) break;
      }
    }
  }
  if (!ok) return decline(TF_MARCH_NO_FIT);
  S->march_declined = TF_MARCH_BUILT;

  // MultiDimensionalSet-layout view: one partition per run, its grid points as first-op ids
  // (the intermediate rows it owns; halo rows it recomputes belong to their own runs), then the
  // same points as fused second-op ids.
  const int nt = (int)S->tiles.size();
  S->ptr1 = {0, nt, nt};
  S->ptr2.assign(nt + 1, 0);
  S->ker_begin.assign(2 * (size_t)nt, 0);
  S->tile_range.resize(4 * (size_t)nt);
  S->writeback.assign(2 * (size_t)nt, 0);
  for (int p = 0; p < nt; ++p) {
    const auto &t = S->tiles[p];
    std::vector<int> own(S->fused_ids.begin() + t.cons_begin, S->fused_ids.begin() + t.cons_end);
    std::sort(own.begin(), own.end());
    for (int r : own) { S->id.push_back(r); S->type.push_back(0); }
    S->ker_begin[2 * p] = (int)S->id.size();
    for (int r : own) { S->id.push_back(r); S->type.push_back(1); }
    S->ker_begin[2 * p + 1] = (int)S->id.size();
    S->ptr2[p + 1] = (int)S->id.size();
    S->tile_range[4 * p + 0] = t.prod_begin; S->tile_range[4 * p + 1] = t.prod_end;
    S->tile_range[4 * p + 2] = t.own_begin;  S->tile_range[4 * p + 3] = t.own_end;
    S->writeback[2 * p] = S->writeback[2 * p + 1] = t.own_begin;
  }
  return true;
}

// Replays every run against the two patterns: what each LDS slot holds in every phase, that each
// ELL row is a row of B (A) entry for entry and in order, that every entry reads a slot which holds
// exactly the row its column names, that nothing is overwritten in the phase that reads it, and that
// every second-op row is computed once.
tf_status validate_march(const tf_schedule *s, int M, const int *Ap, const int *Ai, const int *Bp, const int *Bi) {
  const int n_runs = (int)s->march_runs.size() / 2;
  const int n_slots = (kMaxLds - kMarchSlot0) / kMarchRowBytes;
  if (s->lds_bytes > kMaxLds || s->march_slots > n_slots || s->lds_bytes != kMarchSlot0 + s->march_slots * kMarchRowBytes)
    return fail(TF_ESCHEDULE, "marching schedule: %d bytes of LDS for %d slots", s->lds_bytes, s->march_slots);
  const size_t n_rows = s->march_row_out.size();
  if (s->march_width < 0 || s->march_width > kMarchWideW) return fail(TF_ESCHEDULE, "marching schedule: rows of %d entries", s->march_width);
  const int ell_w = march_ell_stride(s->march_width);
  if (s->march_row_id.size() != n_rows || s->march_ell_off.size() != n_rows * ell_w || s->march_ell_src.size() != n_rows * ell_w ||
      s->march_row_ptr.empty() || s->march_row_ptr.back() != (int)n_rows || s->march_row_ptr.size() != 2 * s->march_load_ptr.size() - 1 ||
      s->march_load_ptr.back() * 2 != (int)s->march_load.size())
    return fail(TF_ESCHEDULE, "marching schedule: tables do not match");
  if (s->march_tpg < 1 || s->march_tpg > kMarchTpg || s->march_dpg < 1 || s->march_dpg > kMarchDpg || s->march_lpg < 1 || s->march_lpg > kMarchLpg)
    return fail(TF_ESCHEDULE, "marching schedule: rows per lane group out of range");
  // the kernel takes only the first march_width pairs of every row
  for (int i = 0; i < M; ++i)
    if (Ap[i + 1] - Ap[i] > s->march_width || Bp[i + 1] - Bp[i] > s->march_width)
      return fail(TF_ESCHEDULE, "marching schedule: row %d has more than the %d entries the schedule says is the most", i, s->march_width);
  const int n_iters = (int)s->march_load_ptr.size() - 1;
  std::vector<int> done(M, 0);
  // slot contents: kind 0 nothing, 1 a row of C, 2 an intermediate row; rstamp/wstamp: the phase (counted
  // over the whole schedule) in which the slot was last read / written
  std::vector<int> kind(n_slots), what(n_slots), rstamp(n_slots, -1), wstamp(n_slots, -1);
  auto slot_of = [&](int off) { return off >= kMarchSlot0 && (off - kMarchSlot0) % kMarchRowBytes == 0 ? (off - kMarchSlot0) / kMarchRowBytes : -1; };
  // the ELL rows [r0, r1) of one phase: their entries against the matrix and against the slots
  auto check_rows = [&](int r, int it, int r0, int r1, bool want_t, int phase) -> tf_status {
    for (int q = r0; q < r1; ++q) {
      const int out = s->march_row_out[q], row = s->march_row_id[q];
      if ((out < 0) != want_t) return fail(TF_ESCHEDULE, "run %d iteration %d: a row of the wrong product in this phase", r, it);
      if (row < 0 || row >= M) return fail(TF_ESCHEDULE, "run %d: row %d out of range", r, row);
      const int *P = want_t ? Bp : Ap, *I = want_t ? Bi : Ai;
      if (!want_t && out != row) return fail(TF_ESCHEDULE, "run %d: second-op row %d is stored to row %d", r, row, out);
      if (P[row + 1] - P[row] > ell_w) return fail(TF_ESCHEDULE, "run %d: row %d has more than %d entries", r, row, ell_w);
      for (int u = 0; u < ell_w; ++u) {
        const int off = s->march_ell_off[(size_t)q * ell_w + u], src = s->march_ell_src[(size_t)q * ell_w + u];
        const int k = P[row] + u;
        if (k >= P[row + 1]) {
          if (off != kMarchZeroOff || src != -1) return fail(TF_ESCHEDULE, "run %d: row %d has an entry past its end", r, row);
          continue;
        }
        if (src != (want_t ? k : (k | kMarchSrcA))) return fail(TF_ESCHEDULE, "run %d: row %d entry %d takes its value from elsewhere", r, row, u);
        const int sl = slot_of(off);
        if (sl < 0 || sl >= s->march_slots) return fail(TF_ESCHEDULE, "run %d: row %d reads outside the slots", r, row);
        if (kind[sl] != (want_t ? 1 : 2) || what[sl] != I[k] || wstamp[sl] >= phase)
          return fail(TF_ESCHEDULE, "run %d iteration %d: row %d of %s reads row %d, which its slot does not hold then", r, it, row,
                      want_t ? "the inner matrix" : "A", I[k]);
        rstamp[sl] = phase;
      }
      if (!want_t && done[row]++) return fail(TF_ESCHEDULE, "second-op row %d scheduled twice", row);
    }
    return TF_OK;
  };
  auto put = [&](int r, int it, int sl, int k, int row, int phase) -> tf_status {
    if (sl < 0 || sl >= s->march_slots) return fail(TF_ESCHEDULE, "run %d iteration %d: a row is stored outside the slots", r, it);
    if (rstamp[sl] == phase) return fail(TF_ESCHEDULE, "run %d iteration %d: a slot is read and overwritten in the same phase", r, it);
    if (wstamp[sl] == phase) return fail(TF_ESCHEDULE, "run %d iteration %d: two rows stored to one slot", r, it);
    kind[sl] = k; what[sl] = row; wstamp[sl] = phase;
    return TF_OK;
  };
  int expect_iter = 0, phase = 0;
  for (int r = 0; r < n_runs; ++r) {
    const int it0 = s->march_runs[2 * r], n_iter = s->march_runs[2 * r + 1];
    if (it0 != expect_iter || n_iter < 1 || n_iter > kMarchMaxIter || it0 + n_iter > n_iters)
      return fail(TF_ESCHEDULE, "run %d: bad iteration range", r);
    expect_iter = it0 + n_iter;
    std::fill(kind.begin(), kind.end(), 0);
    auto loads = [&](int it) -> tf_status {  // list `it` of this run goes to its slots
      const int g = it0 + it, l0 = s->march_load_ptr[g], l1 = s->march_load_ptr[g + 1];
      if (l1 < l0 || (it > 0 && l1 - l0 > s->march_lpg * kMarchGroups)) return fail(TF_ESCHEDULE, "run %d iteration %d: more loads than the lane groups take", r, it);
      for (int q = l0; q < l1; ++q) {
        const int c = s->march_load[2 * q];
        if (c < 0 || c >= M) return fail(TF_ESCHEDULE, "run %d iteration %d: bad load", r, it);
        if (tf_status rc = put(r, it, slot_of(s->march_load[2 * q + 1]), 1, c, phase)) return rc;
      }
      return TF_OK;
    };
    ++phase;
    if (tf_status rc = loads(0)) return rc;  // before the first iteration
    for (int it = 0; it < n_iter; ++it) {
      const int g = it0 + it;
      const int r0 = s->march_row_ptr[2 * g], r1 = s->march_row_ptr[2 * g + 1], r2 = s->march_row_ptr[2 * g + 2];
      if (r1 < r0 || r2 < r1 || r1 - r0 > s->march_tpg * kMarchGroups || r2 - r1 > s->march_dpg * kMarchGroups)
        return fail(TF_ESCHEDULE, "run %d iteration %d: more rows than the lane groups take", r, it);
      ++phase;  // intermediate rows: read slots of C, written to their own
      if (tf_status rc = check_rows(r, it, r0, r1, true, phase)) return rc;
      for (int q = r0; q < r1; ++q)
        if (tf_status rc = put(r, it, slot_of(~s->march_row_out[q]), 2, s->march_row_id[q], phase)) return rc;
      ++phase;  // second-op rows: read slots of the intermediate, while the next rows of C arrive
      if (tf_status rc = check_rows(r, it, r1, r2, false, phase)) return rc;
      if (it + 1 < n_iter)
        if (tf_status rc = loads(it + 1)) return rc;
    }
  }
  if (expect_iter != n_iters) return fail(TF_ESCHEDULE, "marching schedule: iterations left over");
  for (int i = 0; i < M; ++i)
    if (done[i] != 1) return fail(TF_ESCHEDULE, "second-op row %d scheduled %d times", i, done[i]);
  return TF_OK;
}

}  // namespace tf
