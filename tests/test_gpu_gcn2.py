"""tf_gcn_two_layers through two-layer tiles (fused_gcn2_kernel): every tile carries its rows through GEMM, SpMM,
activation, GEMM, SpMM with the hidden layer in LDS.  Held to the oracle's executor composed twice (1e-4 relative,
the GEMMs sum in another order) and, on integer-valued operands, to exact equality."""
import numpy as np
import pytest
import scipy.sparse as sp

from test_gpu_parity import TOL, say

pytestmark = pytest.mark.gpu


def oracle_two_layers(orc, A, X, W1, W2, relu):
    sch = orc.unfused_schedule(A.shape[0])
    h, _ = orc.gemm_spmm(A, X, W1, sch, nthreads=8)
    if relu:
        h = np.maximum(h, 0.0)
    return orc.gemm_spmm(A, h, W2, sch, nthreads=8)[0]


def run_two_layers(tf, Ah, X, W1, W2, s1, s2, relu, fuse, D0=None):
    M, N = X.shape[0], W2.shape[1]
    D = tf.DenseMatrix(M, N, D0) if D0 is not None else tf.DenseMatrix(M, N)
    if D0 is None:
        D.fill(float("nan"))
    tf.gcn_two_layers(Ah, tf.DenseMatrix.from_numpy(X), tf.DenseMatrix.from_numpy(W1), tf.DenseMatrix.from_numpy(W2), D, s1, s2,
                      relu=relu, fuse=fuse, accumulate=D0 is not None)
    tf.device_synchronize()
    return D.to_numpy()


@pytest.mark.parametrize("K,H,N", [(128, 128, 128), (64, 64, 64), (256, 128, 64), (40, 64, 128), (8, 32, 32), (128, 32, 64), (200, 128, 32)])
def test_two_layer_tiles_match_the_oracle(gpu, tf, orc, K, H, N):
    say(f"two-layer tiles K={K} H={H} N={N}")
    M = 20000
    A = tf.workloads.banded_random(M, 32, 16, seed=3)
    Ah = tf.CsrMatrix.from_scipy(A)
    X = tf.workloads.uniform((M, K), 111)
    W1, W2 = tf.workloads.glorot(K, H, 112), tf.workloads.glorot(H, N, 113)
    s1 = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=H, K=K)
    s2 = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=N, K=H)
    s2.validate()
    assert s2.info()["two_layer_tiles"] > 0
    for relu in (True, False):
        want = oracle_two_layers(orc, A, X, W1, W2, relu)
        got = run_two_layers(tf, Ah, X, W1, W2, s1, s2, relu, True)
        assert orc.rel_err(got, want) <= TOL, (K, H, N, relu)
        composed = run_two_layers(tf, Ah, X, W1, W2, s1, s2, relu, False)
        assert orc.rel_err(composed, want) <= TOL
        assert ("fused_gcn2_kernel" in [n for n, _ in _profiled(tf, Ah, X, W1, W2, s1, s2, relu, True)])


def _profiled(tf, Ah, X, W1, W2, s1, s2, relu, fuse):
    s2.set_profiling(True)
    run_two_layers(tf, Ah, X, W1, W2, s1, s2, relu, fuse)
    p = s2.profile()
    s2.set_profiling(False)
    return p


def test_two_layer_tiles_integer_exact_and_accumulate(gpu, tf, orc):
    """Small integers everywhere: every sum is exact in fp32 whatever its order, so the tiles, the composed path and
    the oracle must agree to the bit -- also on a 2D grid (halo of two grid lines), with rows without entries, and when
    D is accumulated into."""
    say("two-layer tiles, integers")
    rng = np.random.default_rng(5)
    band = tf.workloads.banded_random(9000, 32, 16, seed=3)
    band.data = rng.integers(-2, 3, band.nnz).astype(np.float32)
    holes = sp.csr_matrix(sp.diags((rng.random(9000) < 0.8).astype(np.float32)) @ band)
    holes.eliminate_zeros(); holes.sort_indices()
    holes = sp.csr_matrix((holes.data.astype(np.float32), holes.indices.astype(np.int32), holes.indptr.astype(np.int32)), shape=holes.shape)
    grid = tf.workloads.laplacian_2d(64)
    for A, K, H, N in ((band, 64, 64, 64), (holes, 128, 128, 64), (grid, 64, 64, 64)):
        M = A.shape[0]
        Ah = tf.CsrMatrix.from_scipy(A)
        X = rng.integers(-2, 3, (M, K)).astype(np.float32)
        W1 = rng.integers(-1, 2, (K, H)).astype(np.float32)
        W2 = rng.integers(-1, 2, (H, N)).astype(np.float32)
        s1 = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=H, K=K)
        s2 = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=N, K=H)
        s2.validate()
        assert s2.info()["two_layer_tiles"] > 0
        want = oracle_two_layers(orc, A, X, W1, W2, True)
        assert np.abs(want).max() < 2 ** 24
        got = run_two_layers(tf, Ah, X, W1, W2, s1, s2, True, True)
        assert np.array_equal(got, want)
        assert np.array_equal(run_two_layers(tf, Ah, X, W1, W2, s1, s2, True, False), want)
        D0 = rng.integers(-5, 6, (M, N)).astype(np.float32)
        assert np.array_equal(run_two_layers(tf, Ah, X, W1, W2, s1, s2, True, True, D0=D0), want + D0)


def test_two_layer_tiles_full_size_band(gpu, tf, orc):
    """262,144 rows of the banded pattern, K = H = N = 128: against the oracle's executor composed twice."""
    say("two-layer tiles, 262,144-row band")
    cfg = tf.workloads.make_config(6)
    A, X, W1 = cfg["A"], cfg["B"], cfg["C"]
    W2 = tf.workloads.uniform((128, 128), 14)
    Ah = tf.CsrMatrix.from_scipy(A)
    s = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128)
    s.validate()
    info = s.info()
    assert info["two_layer_tiles"] > 0 and info["streamed"] == 1
    want = oracle_two_layers(orc, A, X, W1, W2, True)
    got = run_two_layers(tf, Ah, X, W1, W2, s, s, True, True)
    assert orc.rel_err(got, want) <= TOL
    assert orc.rel_err(run_two_layers(tf, Ah, X, W1, W2, s, s, True, None), want) <= TOL   # the library's own choice


def test_two_layer_tiles_refusals(gpu, tf):
    """TF_FUSE_LAYERS on a schedule without two-layer tiles, or together with a hidden-layer buffer, is refused."""
    cfg = tf.workloads.make_config(3, 0.02)
    A = cfg["A"]
    M = A.shape[0]
    Ah = tf.CsrMatrix.from_scipy(A)
    s = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=64, K=64)
    assert s.info()["two_layer_tiles"] == 0
    X, W = tf.DenseMatrix(M, 64), tf.DenseMatrix(64, 64)
    X.fill(1.0); W.fill(0.5)
    D = tf.DenseMatrix(M, 64)
    with pytest.raises(tf.TileFusionError) as e:
        tf.gcn_two_layers(Ah, X, W, W, D, s, s, fuse=True)
    assert e.value.status == -5
    B = tf.workloads.banded_random(4000, 32, 16, seed=3)
    Bh = tf.CsrMatrix.from_scipy(B)
    sb = tf.inspector(Bh, 1, op=tf.OP_GEMM_SPMM, N=64, K=64)
    Xb, Db, hid = tf.DenseMatrix(4000, 64), tf.DenseMatrix(4000, 64), tf.DenseMatrix(4000, 64)
    Xb.fill(1.0)
    with pytest.raises(tf.TileFusionError) as e:
        tf.gcn_two_layers(Bh, Xb, W, W, Db, sb, sb, fuse=True, hidden=hid)
    assert e.value.status == -5
    tf.gcn_two_layers(Bh, Xb, W, W, Db, sb, sb, hidden=hid)   # composed, hidden layer handed back
    tf.device_synchronize()
    assert np.isfinite(hid.to_numpy()).all()


@pytest.mark.parametrize("lo_off,hi_off,per_row,empty", [(-40, -1, 6, 0.0), (1, 30, 5, 0.1), (-3, 3, 7, 0.3), (-64, 64, 40, 0.05)])
def test_two_layer_tiles_on_bands_off_the_diagonal(gpu, tf, orc, lo_off, hi_off, per_row, empty):
    """Strictly lower and strictly upper bands (a tile's owned rows then lie outside its hidden range), rows without
    entries, rows of 40 entries: the tiles against the oracle composed twice, and exactly on integer operands."""
    from test_inspector import _random_band
    say(f"two-layer tiles, band [{lo_off}, {hi_off}]")
    M, K, H, N = 7000, 64, 64, 64
    A = _random_band(M, lo_off, hi_off, per_row, seed=11, empty_share=empty)
    Ah = tf.CsrMatrix.from_scipy(A)
    s = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=N, K=K, compute_units=16)
    s.validate()
    assert s.info()["two_layer_tiles"] > 0
    X = tf.workloads.uniform((M, K), 131)
    W1, W2 = tf.workloads.glorot(K, H, 132), tf.workloads.glorot(H, N, 133)
    want = oracle_two_layers(orc, A, X, W1, W2, True)
    assert orc.rel_err(run_two_layers(tf, Ah, X, W1, W2, s, s, True, True), want) <= TOL
    rng = np.random.default_rng(6)
    Ai = A.copy(); Ai.data = rng.integers(-2, 3, A.nnz).astype(np.float32)
    Aih = tf.CsrMatrix.from_scipy(Ai)
    Xi = rng.integers(-2, 3, (M, K)).astype(np.float32)
    W1i, W2i = rng.integers(-1, 2, (K, H)).astype(np.float32), rng.integers(-1, 2, (H, N)).astype(np.float32)
    wanti = oracle_two_layers(orc, Ai, Xi, W1i, W2i, True)
    assert np.abs(wanti).max() < 2 ** 24
    assert np.array_equal(run_two_layers(tf, Aih, Xi, W1i, W2i, s, s, True, True), wanti)
