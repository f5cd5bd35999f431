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
