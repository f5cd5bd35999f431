"""The .mtx / .smtx readers (tf_read_matrix, tf_read_dense) against scipy.io.mmread -- an
independent implementation of the published MatrixMarket format -- and against hand-written
files; exact comparison (values are fp32 of the file's numbers)."""
import numpy as np
import pytest
import scipy.io as sio
import scipy.sparse as sp


def same_csr(got, want):
    want = sp.csr_matrix(want, dtype=np.float64)
    want.sum_duplicates()
    want.sort_indices()
    got = got.copy()
    assert got.shape == want.shape
    assert got.has_sorted_indices or np.all(np.diff(got.indices) != 0)
    assert np.array_equal(got.indptr, want.indptr) and np.array_equal(got.indices, want.indices)
    assert np.array_equal(got.data, want.data.astype(np.float32))


@pytest.mark.parametrize("kind", ["general", "symmetric", "skew", "pattern", "integer", "rectangular", "empty_rows"])
def test_mtx_matches_scipy(tf, tmp_path, kind):
    rng = np.random.default_rng(hash(kind) % 1000)
    n = 60
    A = sp.random(n, n, density=0.08, random_state=rng.integers(1 << 30), format="coo", dtype=np.float64)
    A.data = np.round(A.data * 100) / 8.0 + 0.125
    path = str(tmp_path / f"{kind}.mtx")
    if kind == "symmetric":
        A = (A + A.T).tocoo()
        sio.mmwrite(path, A, symmetry="symmetric")
    elif kind == "skew":
        A = (A - A.T).tocoo()
        sio.mmwrite(path, A, symmetry="skew-symmetric")
    elif kind == "pattern":
        sio.mmwrite(path, A, field="pattern")
    elif kind == "integer":
        A.data = np.round(A.data * 8)
        sio.mmwrite(path, A.astype(np.int64), field="integer")
    elif kind == "rectangular":
        A = sp.random(40, 90, density=0.1, random_state=7, format="coo", dtype=np.float64)
        sio.mmwrite(path, A)
    elif kind == "empty_rows":
        A = A.tolil()
        A[5] = 0
        A[17] = 0
        A = A.tocoo()
        sio.mmwrite(path, A)
    else:
        sio.mmwrite(path, A)
    same_csr(tf.read_matrix(path), sio.mmread(path))


def test_mtx_by_hand_with_comments_duplicates_and_symmetry(tf, tmp_path):
    path = tmp_path / "hand.mtx"
    path.write_text("%%MatrixMarket matrix coordinate real symmetric\n% a comment\n\n%another\n4 4 5\n"
                    "1 1 2.5\n3 1 -1\n3 1 0.5\n4 2 7\n4 4 1e-1\n")
    got = tf.read_matrix(str(path)).toarray()
    want = np.zeros((4, 4), np.float32)
    want[0, 0] = 2.5
    want[2, 0] = want[0, 2] = -0.5  # the two (3,1) entries add up
    want[3, 1] = want[1, 3] = 7
    want[3, 3] = np.float32(0.1)
    assert np.array_equal(got, want)


def test_smtx(tf, tmp_path):
    """DLMC format as the reference reads it (Fusion_Utils.cpp:205-250): values are all 1."""
    path = tmp_path / "m.smtx"
    path.write_text("3, 5, 6\n0 2 2 6\n4 1\n0 1 2 3\n")
    got = tf.read_matrix(str(path))
    assert got.shape == (3, 5) and got.indptr.tolist() == [0, 2, 2, 6]
    assert got.indices.tolist() == [1, 4, 0, 1, 2, 3] and np.all(got.data == 1.0)


def test_dense_array_file(tf, tmp_path):
    rng = np.random.default_rng(3)
    X = np.round(rng.uniform(-4, 4, (7, 5)) * 16) / 16
    path = str(tmp_path / "x.mtx")
    sio.mmwrite(path, X)
    assert np.array_equal(tf.read_dense(path), X.astype(np.float32))
    S = X[:5, :5] + X[:5, :5].T
    sio.mmwrite(path, S, symmetry="symmetric")
    assert np.array_equal(tf.read_dense(path), S.astype(np.float32))


def test_reader_errors(tf, tmp_path):
    with pytest.raises(tf.TileFusionError, match="cannot open"):
        tf.read_matrix(str(tmp_path / "missing.mtx"))
    p = tmp_path / "x.csv"
    p.write_text("1,2,3\n")
    with pytest.raises(tf.TileFusionError, match="extension"):
        tf.read_matrix(str(p))
    p = tmp_path / "bad.mtx"
    p.write_text("%%MatrixMarket matrix coordinate real general\n3 3 2\n1 1 1.0\n")
    with pytest.raises(tf.TileFusionError, match="end early"):
        tf.read_matrix(str(p))
    p.write_text("%%MatrixMarket matrix coordinate real general\n3 3 1\n4 1 1.0\n")
    with pytest.raises(tf.TileFusionError, match="out of range"):
        tf.read_matrix(str(p))
    p.write_text("%%MatrixMarket matrix coordinate complex general\n1 1 1\n1 1 1.0 0.0\n")
    with pytest.raises(tf.TileFusionError, match="complex"):
        tf.read_matrix(str(p))
    p = tmp_path / "bad.smtx"
    p.write_text("2, 2, 3\n0 1 2\n0 1\n")
    with pytest.raises(tf.TileFusionError, match="span"):
        tf.read_matrix(str(p))
