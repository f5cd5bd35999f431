"""The synthetic operand generators, pinned by hand-computed cases and by the properties the
configurations are defined through.  CPU only."""
import numpy as np
import scipy.sparse as sp


def test_gcn_normalise_five_node_graph(tf):
    """x_ij / sqrt(deg_i * deg_j), deg = stored entries per row with the self-loops in
    (normalizeAdjacencyMatrix, GCN_Single_Layer_SP_Demo_Utils.h:40-53), on a path 0-1-2 with a
    pendant 3 on node 1 and an isolated node 4, worked out by hand:
        deg = [2, 4, 2, 2, 1]
        row 0: (0,0) 1/2          (0,1) 1/sqrt(8)
        row 1: (1,0) 1/sqrt(8)    (1,1) 1/4   (1,2) 1/sqrt(8)   (1,3) 1/sqrt(8)
        row 2: (2,1) 1/sqrt(8)    (2,2) 1/2
        row 3: (3,1) 1/sqrt(8)    (3,3) 1/2
        row 4: (4,4) 1
    """
    edges = [(0, 1), (1, 2), (1, 3)]
    a = np.eye(5)
    for u, v in edges:
        a[u, v] = a[v, u] = 1.0
    got = tf.workloads.gcn_normalise(sp.csr_matrix(a)).toarray()
    r8 = 1.0 / np.sqrt(8.0)
    want = np.array([[0.5, r8, 0, 0, 0],
                     [r8, 0.25, r8, r8, 0],
                     [0, r8, 0.5, 0, 0],
                     [0, r8, 0, 0.5, 0],
                     [0, 0, 0, 0, 1.0]], np.float32)
    assert got.dtype == np.float32
    assert np.allclose(got, want, rtol=0, atol=1e-7)
    # values other than 1 scale through, and the degree is the entry count, not the row sum
    b = a.copy()
    b[0, 1] = 3.0
    got = tf.workloads.gcn_normalise(sp.csr_matrix(b)).toarray()
    assert np.isclose(got[0, 1], 3.0 * r8) and np.isclose(got[1, 0], r8)


def test_erdos_renyi_gcn_is_symmetric_normalised(tf):
    A = tf.workloads.erdos_renyi_gcn(3000, 10.0, seed=5)
    assert A.indices.dtype == np.int32 and A.data.dtype == np.float32 and A.has_sorted_indices
    assert (A.diagonal() > 0).all()                       # self-loops
    assert abs(A - A.T).max() < 1e-7                      # symmetric
    deg = np.diff(A.indptr).astype(np.float64)
    # undo the normalisation: every stored entry was 1
    ones = sp.diags(np.sqrt(deg)) @ A.astype(np.float64) @ sp.diags(np.sqrt(deg))
    assert np.allclose(ones.data, 1.0, atol=1e-5)
    assert 9.0 < (deg.mean() - 1.0) < 11.0                # mean degree 10 plus the self-loop


def test_rmat_rows_sum_to_one_and_are_skewed(tf):
    A = tf.workloads.rmat(14, (1 << 14) * 8, seed=8)
    assert A.shape == (1 << 14, 1 << 14) and A.indices.dtype == np.int32 and A.has_sorted_indices
    sums = np.asarray(A.sum(axis=1)).ravel()
    nonempty = np.diff(A.indptr) > 0
    assert np.allclose(sums[nonempty], 1.0, atol=1e-5)    # row-normalised
    assert (sums[~nonempty] == 0).all()
    pattern = sp.csr_matrix((np.ones(A.nnz), A.indices, A.indptr), shape=A.shape)
    assert abs(pattern - pattern.T).max() == 0            # symmetrised
    deg = np.diff(A.indptr)
    assert deg.max() > 50 * max(1.0, np.median(deg[nonempty]))   # power law: hubs
    assert (~nonempty).mean() > 0.2                        # and many isolated nodes
    # every row's values are equal (1 / degree)
    row = np.repeat(np.arange(A.shape[0]), deg)
    assert np.allclose(A.data * deg[row], 1.0, atol=1e-5)


def test_laplacians_and_band(tf):
    w = tf.workloads
    A = w.laplacian_2d(5, 4)
    assert A.nnz == 5 * 20 - 2 * (5 + 4) and (A.diagonal() == 4).all()
    assert (np.asarray(A.sum(axis=1)).ravel() == 4 - (np.diff(A.indptr) - 1)).all()
    A = w.laplacian_3d(6)
    assert A.nnz == 7 * 216 - 6 * 36 and (A.diagonal() == 6).all()
    # x fastest: row 1 couples to 0, 2 (x), 7 (y), 37 (z)
    assert A[1].indices.tolist() == [0, 1, 2, 7, 37]
    A = w.banded_random(500, 32, 16, seed=3)
    r = np.repeat(np.arange(500), np.diff(A.indptr))
    assert ((A.indices - r >= -16) & (A.indices - r < 16)).all()
    assert (np.diff(A.indptr)[16:-16] == 16).all()
