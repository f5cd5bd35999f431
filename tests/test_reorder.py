"""tf_reorder_rcm / tf_permute_csr: the library form of the reference's offline reordering
(scripts/reorder_graphs.py:21-22: scipy's reverse_cuthill_mckee, then A[perm,:][:,perm]).
Pinned by what the mathematics fixes -- perm is a permutation, the permuted matrix is the
scipy fancy-indexing result, a scrambled band gets its bandwidth back -- and by scipy's own
RCM as an independent implementation (bandwidth within a small factor; the two need not
pick the same permutation).  Host-only tests."""
import numpy as np
import pytest
import scipy.sparse as sp
from scipy.sparse.csgraph import reverse_cuthill_mckee


def bandwidth(A):
    A = sp.coo_matrix(A)
    return int(np.abs(A.row - A.col).max()) if A.nnz else 0


def scrambled(A, seed):
    p = np.random.default_rng(seed).permutation(A.shape[0])
    return sp.csr_matrix(A[p, :][:, p]), p


def test_rcm_restores_a_scrambled_band(tf):
    A = tf.workloads.banded_random(6000, 32, 16, seed=1)
    S, _ = scrambled(A, 2)
    assert bandwidth(S) > 4000
    perm = tf.reorder_rcm(S)
    assert np.array_equal(np.sort(perm), np.arange(6000))
    R = tf.permute_csr(S, perm)
    ref = sp.csr_matrix(S[perm, :][:, perm])
    ref.sort_indices()
    assert np.array_equal(R.indptr, ref.indptr) and np.array_equal(R.indices, ref.indices) and np.array_equal(R.data, ref.data)
    theirs = reverse_cuthill_mckee(sp.csr_matrix(S), symmetric_mode=False)
    bw_theirs = bandwidth(S[theirs, :][:, theirs])
    assert bandwidth(R) <= 2 * bandwidth(A) + 8
    assert bandwidth(R) <= 1.25 * bw_theirs + 8


def test_rcm_grid_and_components(tf):
    # a 2D grid scrambled: bandwidth back to the order of the grid's side
    G, _ = scrambled(tf.workloads.laplacian_2d(60), 3)
    perm = tf.reorder_rcm(G)
    assert bandwidth(tf.permute_csr(G, perm)) <= 2 * 60 + 4
    # two components, isolated nodes, an unsymmetric pattern, an explicit diagonal
    B = sp.block_diag([tf.workloads.banded_random(300, 8, 4, seed=4), sp.csr_matrix((5, 5), dtype=np.float32),
                       sp.triu(tf.workloads.laplacian_2d(12))], format="csr", dtype=np.float32)
    S, _ = scrambled(B, 5)
    perm = tf.reorder_rcm(S)
    assert np.array_equal(np.sort(perm), np.arange(B.shape[0]))
    R = tf.permute_csr(S, perm)
    assert bandwidth(R) <= 40 and R.nnz == B.nnz
    assert abs(R.sum() - B.sum()) < 1e-3
    # nothing to do / empty
    assert tf.reorder_rcm(sp.csr_matrix((0, 0), dtype=np.float32)).shape == (0,)
    E = sp.identity(7, format="csr", dtype=np.float32)
    assert np.array_equal(np.sort(tf.reorder_rcm(E)), np.arange(7))


def test_rcm_makes_a_scrambled_band_fuse(tf):
    """What the reordering is for: the scrambled matrix fuses nothing, the reordered one gets
    windowed tiles that fuse every row."""
    A = tf.workloads.banded_random(8192, 32, 16, seed=6)
    S, _ = scrambled(A, 7)
    Sh = tf.CsrMatrix.from_scipy(S)
    before = tf.inspector(Sh, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Sh).info()
    R = tf.permute_csr(S, tf.reorder_rcm(S))
    Rh = tf.CsrMatrix.from_scipy(R)
    sched = tf.inspector(Rh, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Rh)
    sched.validate()
    after = sched.info()
    assert before["n_fused_rows"] < 0.05 * 8192
    assert after["n_fused_rows"] == 8192 and after["windowed"] == 1


def test_bad_arguments(tf):
    A = sp.csr_matrix(np.ones((3, 4), np.float32))
    with pytest.raises(ValueError):
        tf.reorder_rcm(A)
    B = tf.workloads.banded_random(50, 4, 2, seed=8)
    with pytest.raises(tf.TileFusionError):
        tf.permute_csr(B, np.zeros(50, np.int32))
    with pytest.raises(ValueError):
        tf.permute_csr(B, np.arange(49))


def _cut_fraction(A, perm, part_ptr):
    """Share of the off-diagonal entries whose two ends lie in different parts (hubs count as a part of their own)."""
    M = A.shape[0]
    part_of_new = np.searchsorted(part_ptr[1:], np.arange(M), side="right")
    part = np.empty(M, int)
    part[perm] = part_of_new
    C = sp.coo_matrix(A)
    off = C.row != C.col
    return float((part[C.row[off]] != part[C.col[off]]).mean())


def test_partition_ordering_cuts_few_edges_of_a_grid(tf):
    """tf_reorder_partition on a scrambled 2D grid: a permutation, parts of equal size, and compact parts -- a small
    share of the edges crosses between parts (16 random parts of a grid cut 15/16 of them; square blocks of a 96 x 96
    grid cut about 1/12).  The permuted matrix equals scipy's fancy indexing, as for RCM."""
    n = 96
    G, _ = scrambled(tf.workloads.laplacian_2d(n), 7)
    perm, pp = tf.reorder_partition(G, 16)
    M = n * n
    assert np.array_equal(np.sort(perm), np.arange(M))
    assert pp[0] == 0 and pp[1] == 0 and pp[-1] == M           # a grid has no hubs
    sizes = np.diff(pp[1:])
    assert sizes.min() >= M // 16 and sizes.max() <= M // 16 + 1
    cut = _cut_fraction(G, perm, pp)
    assert cut < 0.2, cut
    rnd = np.random.default_rng(1).permutation(M).astype(np.int32)
    assert _cut_fraction(G, rnd, pp) > 0.9                      # the measure itself: random parts cut nearly all
    R = tf.permute_csr(G, perm)
    ref = sp.csr_matrix(G[perm, :][:, perm]); ref.sort_indices()
    assert np.array_equal(R.indptr, ref.indptr) and np.array_equal(R.indices, ref.indices)


def test_partition_ordering_sets_hubs_aside(tf):
    """On a power-law graph the vertices of very high degree come first, by falling degree, and the rest is still
    dealt into equal parts; isolated vertices, several components and one part are handled."""
    cfg = tf.workloads.make_config(4, 2.0 ** -7)
    A = cfg["A"]
    M = A.shape[0]
    S = sp.csr_matrix(A + A.T)
    deg = np.diff(S.indptr) - (S.diagonal() != 0)
    perm, pp = tf.reorder_partition(A, 8)
    assert np.array_equal(np.sort(perm), np.arange(M))
    nh = pp[1]
    thr = max(64, 16 * (deg.sum() // M))
    assert nh == int((deg > thr).sum()) > 0
    assert np.all(np.diff(deg[perm[:nh]]) <= 0) and deg[perm[:nh]].min() > thr and deg[perm[nh:]].max() <= thr
    sizes = np.diff(pp[1:])
    assert sizes.max() - sizes.min() <= 1 and pp[-1] == M
    perm1, pp1 = tf.reorder_partition(A, 1, hub_degree=10 ** 9)   # no hubs, one part: still a permutation
    assert pp1[1] == 0 and np.array_equal(np.sort(perm1), np.arange(M))
    B = sp.block_diag([tf.workloads.laplacian_2d(10), sp.csr_matrix((6, 6), dtype=np.float32), tf.workloads.laplacian_2d(7)], format="csr")
    permb, ppb = tf.reorder_partition(B, 4)
    assert np.array_equal(np.sort(permb), np.arange(B.shape[0])) and ppb[-1] == B.shape[0]
    with pytest.raises(tf.TileFusionError):
        tf.reorder_partition(A, 0)
