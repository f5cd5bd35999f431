"""Pins the C restatement of the reference inspectors (oracle/tf_oracle.c): hand-derived
golden schedules, structural closed forms on banded patterns, and the invariants every
reference schedule obeys.  CPU only."""
import json
import os

import numpy as np
import pytest
import scipy.sparse as sp

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tridiag8_schedules.json")


def banded_pattern(M, h):
    """Row i stores every column in [i-h, i+h] clipped to the matrix."""
    diags = [np.ones(M - abs(k)) for k in range(-h, h + 1)]
    return sp.csr_matrix(sp.diags(diags, list(range(-h, h + 1)), format="csr"))


def check_reference_invariants(S, A):
    """What every schedule of the reference's format must satisfy (layout filled at
    Fusion_Inspector.h:959-1010): each first-op row once, each second-op row once, tiles
    contiguous and ascending, fused rows depend only on their tile's first-op rows,
    pointer arrays consistent."""
    M = A.shape[0]
    assert S.ptr1[0] == 0 and S.ptr2[0] == 0
    P = S.ptr1[S.n1]
    assert len(S.ptr2) == P + 1 and np.all(np.diff(S.ptr2) >= 0)
    assert S.ptr2[P] == len(S.id) == 2 * M
    first = S.id[S.type == 0]
    second = S.id[S.type == 1]
    assert np.array_equal(np.sort(first), np.arange(M))
    assert np.array_equal(np.sort(second), np.arange(M))
    lvl0, lvl1 = S.tiles()
    end = 0
    for p, (rows, fused) in enumerate(lvl0):
        assert len(rows) > 0 and rows[0] == end and np.array_equal(rows, np.arange(rows[0], rows[0] + len(rows)))
        end = rows[-1] + 1
        assert S.ker_begin[2 * p + 1] == S.ptr2[p + 1]
        for i in fused:
            cols = A.indices[A.indptr[i]:A.indptr[i + 1]]
            assert cols.min() >= rows[0] and cols.max() <= rows[-1], f"fused row {i} leaves tile {p}"
    assert end == M
    for q, rows in enumerate(lvl1):
        p = S.ptr1[1] + q
        assert S.ker_begin[2 * p] == S.ptr2[p] and S.ker_begin[2 * p + 1] == S.ptr2[p + 1]
    rem = np.concatenate(lvl1) if lvl1 else np.zeros(0, np.int32)
    return lvl0, rem


@pytest.fixture(scope="module")
def gold():
    with open(GOLD) as f:
        return json.load(f)


def _pattern(g):
    p = g["pattern"]
    M = p["M"]
    return sp.csr_matrix((np.ones(len(p["indices"])), np.array(p["indices"]), np.array(p["indptr"])), shape=(M, M))


@pytest.mark.parametrize("which", ["vt_gemm_spmm", "vt_both_wavefronts", "fixed_tiles"])
def test_hand_derived_schedule(orc, gold, which):
    A = _pattern(gold)
    g = gold[which]
    a = g["args"]
    if which == "vt_gemm_spmm":
        S = orc.inspect_vt_gemm_spmm(A, a["BCol"], a["CCol"], a["cache"], a["DataSize"])
    elif which == "vt_both_wavefronts":
        S = orc.inspect_vt_both_wavefronts(A, a["BCol"], a["cache"], a["NumThreads"], a["DataSize"])
    else:
        S = orc.inspect_fixed_tiles(A, a["IterPerPartition"], a["NumThreads"])
    assert S.n1 == g["n1"]
    for name in ("ptr1", "ptr2", "ker_begin", "id", "type"):
        assert getattr(S, name).tolist() == g[name], name


@pytest.mark.parametrize("M,h,K,N,cache", [(1024, 1, 32, 32, 40000), (4096, 16, 64, 64, 100000), (3000, 5, 32, 64, 60000)])
def test_vt_gemm_banded_closed_form(orc, M, h, K, N, cache):
    """Full band of half-width h: the fused rows of a tile [s,e) are exactly
    [s+h, e-h) (clipped at the matrix ends), so the remainder is the 2h rows around every
    interior tile boundary; every final tile fits the cache model and none could have
    stayed at twice its size (the halving rule, Fusion_Inspector.h:894-923)."""
    A = banded_pattern(M, h)
    S = orc.inspect_vt_gemm_spmm(A, K, N, cache)
    lvl0, rem = check_reference_invariants(S, A)
    nnz_row = np.diff(A.indptr)

    def ws(s, e):  # Fusion_Inspector.h:1025-1027 on the closed-form fused set
        f0 = s if s == 0 else s + h
        f1 = e if e == M else e - h
        nf = max(0, f1 - f0)
        fnnz = int(nnz_row[f0:f1].sum()) if nf else 0
        return ((e - s) * N + N * K + (e - s) * K + nf * N + fnnz) * 4 + fnnz * 4

    initial = min((cache // 4 - K * N) // (K + N), M)
    expected_rem = []
    for rows, fused in lvl0:
        s, e = rows[0], rows[-1] + 1
        f0 = s if s == 0 else s + h
        f1 = e if e == M else e - h
        assert np.array_equal(fused, np.arange(f0, max(f0, f1)))
        expected_rem += [r for r in range(s, e) if not (f0 <= r < f1)]
        assert ws(s, e) <= cache or e - s == 1
        if e - s < initial:  # produced by a split: its parent must have been too big
            assert ws(s, min(M, s + 2 * (e - s))) > cache or ws(max(0, e - 2 * (e - s)), e) > cache
    assert np.array_equal(rem, np.array(sorted(expected_rem), dtype=np.int32))


@pytest.mark.parametrize("threads", [1, 4, 8])
def test_vt_both_wavefronts_invariants(orc, tf, threads):
    A = tf.workloads.banded_random(4096, 32, 16, seed=11)
    S = orc.inspect_vt_both_wavefronts(A, 64, 100000, threads)
    lvl0, rem = check_reference_invariants(S, A)
    assert np.all(np.diff(rem) > 0)  # remainder rows are sorted (Fusion_Inspector.h:754)
    cap = min(4096, A.shape[0] // (2 * threads))
    assert max(len(r) for r, _ in lvl0) <= cap + 1


def test_fixed_tiles_invariants(orc, tf):
    A = tf.workloads.laplacian_2d(32)
    for ipp, threads in [(64, 1), (128, 2), (2048, 4)]:
        S = orc.inspect_fixed_tiles(A, ipp, threads)
        lvl0, rem = check_reference_invariants(S, A)
        nparts = max(A.shape[0] // ipp, 2 * threads)
        assert len(lvl0) == nparts
        sizes = [len(r) for r, _ in lvl0]
        assert max(sizes) == -(-A.shape[0] // nparts)
        # 5-point stencil on a 32-wide grid: a row fuses iff rows i-32 and i+32 (where they exist) are in its tile
        for rows, fused in lvl0:
            s, e = rows[0], rows[-1] + 1
            want = [i for i in range(s, e) if (i - 32 < 0 or i - 32 >= s) and (i + 32 >= A.shape[0] or i + 32 < e)
                    and (i % 32 == 0 or i - 1 >= s) and (i % 32 == 31 or i + 1 < e)]
            assert fused.tolist() == want


def test_fused_stats_and_errors(orc):
    import ctypes as C
    A = banded_pattern(256, 2)
    S = orc.inspect_vt_gemm_spmm(A, 32, 32, 30000)
    lvl0, _ = S.tiles()
    n_fused = sum(len(f) for _, f in lvl0)
    assert n_fused == int(((S.type == 1) & (np.arange(len(S.id)) < S.ptr2[S.ptr1[1]])).sum())
    # a cache too small for even K*N makes the reference's initial tile non-positive: reported, not run
    with pytest.raises(ValueError):
        orc.inspect_vt_gemm_spmm(A, 128, 128, 60000)


def test_empty_rows_do_not_read_outside(orc):
    """The reference reads Ai[Ap[i]] on empty rows; the restatement treats them as fused."""
    M = 64
    A = sp.lil_matrix((M, M))
    for i in range(0, M, 2):
        A[i, i] = 1.0
    A = sp.csr_matrix(A)
    S = orc.inspect_vt_gemm_spmm(A, 32, 32, 20000)
    lvl0, rem = S.tiles()
    assert sum(len(f) for _, f in lvl0) == M and sum(len(r) for r in rem) == 0
