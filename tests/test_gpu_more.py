"""More parity cases on the GPU, through the C ABI: operands that arrive as files, schedules
handed the wrong operands, the full-size GCN layer, launches timed one by one."""
import numpy as np
import pytest
import scipy.io
import scipy.sparse as sp

from test_gpu_parity import TOL, oracle_spmm_spmm, say

pytestmark = pytest.mark.gpu


def test_matrix_files_through_both_executors(gpu, tf, orc, tmp_path):
    """A symmetric MatrixMarket file (lower triangle stored, expanded as the reference's drivers
    do with make_full) and a DLMC .smtx file (pattern only, every value 1) are read by
    tf_read_matrix, run through both executors and compared with the oracle on the matrix that
    scipy reads from the same file / that the file was written from."""
    say("files: .mtx symmetric + .smtx -> HIP -> oracle")
    n = 48
    L = tf.workloads.laplacian_2d(n)                       # symmetric, 2304 rows
    rng = np.random.default_rng(81)
    L.data = L.data * rng.uniform(0.5, 1.5, L.nnz).astype(np.float32)
    L = sp.csr_matrix((L + L.T) * 0.5, dtype=np.float32)   # symmetric values
    mtx = tmp_path / "lap.mtx"
    scipy.io.mmwrite(str(mtx), sp.tril(L).tocoo(), symmetry="symmetric", precision=9)
    G = tf.workloads.banded_random(3000, 32, 12, seed=82)
    smtx = tmp_path / "band.smtx"
    with open(smtx, "w") as f:
        f.write(f"{G.shape[0]}, {G.shape[1]}, {G.nnz}\n")
        f.write(" ".join(map(str, G.indptr)) + "\n")
        f.write(" ".join(map(str, G.indices)) + "\n")
    want_mtx = sp.csr_matrix(scipy.io.mmread(str(mtx)), dtype=np.float32)
    want_mtx.sort_indices()
    want_smtx = sp.csr_matrix((np.ones(G.nnz, np.float32), G.indices, G.indptr), shape=G.shape)
    for path, ref in ((mtx, want_mtx), (smtx, want_smtx)):
        A = tf.read_matrix(path)
        assert A.shape == ref.shape and np.array_equal(A.indptr, ref.indptr) and np.array_equal(A.indices, ref.indices)
        assert np.array_equal(A.data, ref.data)
        M = A.shape[0]
        Ah = tf.CsrMatrix.from_scipy(A)
        # SpMM-SpMM, bit for bit
        Cd = tf.workloads.uniform((M, 64), 83)
        S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Ah)
        S.validate()
        D = tf.DenseMatrix(M, 64)
        tf.spmm_spmm(Ah, Ah, tf.DenseMatrix.from_numpy(Cd), D, S)
        assert np.array_equal(D.to_numpy(), oracle_spmm_spmm(orc, ref, ref, Cd)), path
        # GeMM-SpMM, 1e-4
        B, W = tf.workloads.uniform((M, 40), 84), tf.workloads.uniform((40, 64), 85)
        S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=64, K=40)
        S.validate()
        D = tf.DenseMatrix(M, 64)
        tf.gemm_spmm(Ah, tf.DenseMatrix.from_numpy(B), tf.DenseMatrix.from_numpy(W), D, S)
        want, _ = orc.gemm_spmm(ref, B, W, orc.unfused_schedule(M))
        assert orc.rel_err(D.to_numpy(), want) <= TOL, path


def test_schedule_refuses_another_pattern(gpu, tf, orc):
    """The windowed kernels turn B's columns into LDS offsets inside a tile's window, and every
    kernel trusts the schedule's row lists: operands with the right shape and entry count but
    another pattern are refused (TF_ESCHEDULE), for A and for B, on the wide and the lane-group
    windowed kernels.  A wrapped matrix is checked once its owner provides the fingerprint."""
    say("pattern fingerprints")
    M, N = 4000, 128
    A = tf.workloads.banded_random(M, 32, 16, seed=3)
    X = tf.workloads.banded_random(M, 32, 16, seed=9)      # same shape, same nnz, other pattern
    assert X.nnz == A.nnz
    Ah, Xh = tf.CsrMatrix.from_scipy(A), tf.CsrMatrix.from_scipy(X)
    Cd = tf.DenseMatrix.from_numpy(tf.workloads.uniform((M, N), 86))
    D = tf.DenseMatrix(M, N)
    for kw in (dict(), dict(wide_strips=-1, strip_cols=32)):
        S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=N, inner=Ah, **kw)
        assert S.info()["windowed"] == 1
        for a, b in ((Ah, Xh), (Xh, Ah), (Xh, Xh)):
            with pytest.raises(tf.TileFusionError) as e:
                tf.spmm_spmm(a, b, Cd, D, S)
            assert e.value.status == -4 and "pattern" in str(e.value)
        tf.spmm_spmm(Ah, Ah, Cd, D, S)                      # the right operands still run
    S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=64, K=64)
    B = tf.DenseMatrix.from_numpy(tf.workloads.uniform((M, 64), 87))
    W = tf.DenseMatrix.from_numpy(tf.workloads.uniform((64, 64), 88))
    D = tf.DenseMatrix(M, 64)
    with pytest.raises(tf.TileFusionError) as e:
        tf.gemm_spmm(Xh, B, W, D, S)
    assert e.value.status == -4


def test_gcn_layer_full_size_all_ones_features(gpu, tf):
    """The GCN-layer configuration at full size (200,000 nodes, K = 256, N = 128): with all-ones
    features every row of the intermediate is the column sums of the weights, so
    D = rowsum(A) * colsum(C)^T -- a check that needs no oracle run at this size."""
    say("gemm_spmm GCN layer 200k nodes, B = ones")
    cfg = tf.workloads.make_config(3)
    A, W = cfg["A"], cfg["C"]
    M, K, N = A.shape[0], cfg["K"], cfg["N"]
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=N, K=K)
    S.validate()
    B = tf.DenseMatrix(M, K); B.fill(1.0)
    D = tf.DenseMatrix(M, N); D.fill(float("nan"))
    tf.gemm_spmm(Ah, B, tf.DenseMatrix.from_numpy(W), D, S)
    tf.device_synchronize()
    want = np.asarray(A.astype(np.float64).sum(axis=1)) * W.astype(np.float64).sum(axis=0)[None, :]
    got = D.to_numpy()
    assert np.abs(got - want).max() / np.abs(want).max() <= TOL
    # and with the configuration's own features, against fp64 on a sample of rows
    D.fill(float("nan"))
    tf.gemm_spmm(Ah, tf.DenseMatrix.from_numpy(cfg["B"]), tf.DenseMatrix.from_numpy(W), D, S)
    rows = np.random.default_rng(89).choice(M, 4096, replace=False)
    T = cfg["B"].astype(np.float64) @ W.astype(np.float64)
    want = A[rows].astype(np.float64) @ T
    assert np.abs(D.to_numpy()[rows] - want).max() / np.abs(want).max() <= TOL


def test_launch_times_and_second_stream(gpu, tf, orc):
    """tf_schedule_set_profiling: every launch of a call is timed; and a power-law product run
    on one stream and with the hot segments on the executor's second stream (TF_SECOND_STREAM)
    gives the same bits (the summation order is fixed by the schedule, not by timing)."""
    say("per-launch times, second stream")
    cfg = tf.workloads.make_config(4, 2.0 ** -5)
    A, B, W = cfg["A"], cfg["B"], cfg["C"]
    M = A.shape[0]
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128, long_row_partition=1)
    S.validate()
    assert S.info()["long_row_hot_cols"] > 0
    Bd, Wd = tf.DenseMatrix.from_numpy(B), tf.DenseMatrix.from_numpy(W)
    D1, D2 = tf.DenseMatrix(M, 128), tf.DenseMatrix(M, 128)
    S.set_profiling(True)
    tf.gemm_spmm(Ah, Bd, Wd, D1, S)
    prof1 = S.profile()
    tf.gemm_spmm(Ah, Bd, Wd, D2, S, second_stream=True)
    prof2 = S.profile()
    S.set_profiling(False)
    tf.device_synchronize()
    assert len(prof1) >= 4 and all(ms > 0 for _, ms in prof1), prof1
    assert any("hot long-row segments" in n for n, _ in prof2), prof2
    assert any("hot rows" in n for n, _ in prof2), prof2
    a, b = D1.to_numpy(), D2.to_numpy()
    assert np.array_equal(a, b)
    want, _ = orc.gemm_spmm(A, B, W, orc.unfused_schedule(M), nthreads=8)
    assert orc.rel_err(a, want) <= TOL
    for _ in range(3):                                       # replays keep giving the same bits
        tf.gemm_spmm(Ah, Bd, Wd, D2, S)
        assert np.array_equal(D2.to_numpy(), a)


def test_second_stream_on_a_first_call_and_on_wrapped_matrices(gpu, tf, orc):
    """TF_SECOND_STREAM when the regrouped values of the long rows have to be built in the same call: on the
    first call with a fresh schedule, and on every call with a matrix wrapped around device arrays (whose
    values the library takes as new each time).  The cold segments run on the caller's stream and read values
    the same call regroups, so that copy has to come before the fork: results must equal the one-stream
    call's bit for bit, also after the wrapped matrix' values changed in place."""
    say("second stream: first call, wrapped matrix")
    cfg = tf.workloads.make_config(4, 2.0 ** -5)
    A, B, W = cfg["A"], cfg["B"], cfg["C"]
    M = A.shape[0]
    Bd, Wd = tf.DenseMatrix.from_numpy(B), tf.DenseMatrix.from_numpy(W)
    Ah = tf.CsrMatrix.from_scipy(A)
    S0 = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128, long_row_partition=1)
    D0 = tf.DenseMatrix(M, 128)
    tf.gemm_spmm(Ah, Bd, Wd, D0, S0)
    want = D0.to_numpy()
    # a fresh schedule whose first call already forks
    S1 = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128, long_row_partition=1)
    D1 = tf.DenseMatrix(M, 128); D1.fill(float("nan"))
    tf.gemm_spmm(Ah, Bd, Wd, D1, S1, second_stream=True)
    assert np.array_equal(D1.to_numpy(), want)
    # the same matrix wrapped around device arrays: values regrouped on every call
    as_f32 = lambda a: np.ascontiguousarray(a, dtype=np.int32).view(np.float32).reshape(1, -1)  # noqa: E731
    dp, di = tf.DenseMatrix.from_numpy(as_f32(A.indptr)), tf.DenseMatrix.from_numpy(as_f32(A.indices))
    dx = tf.DenseMatrix.from_numpy(A.data.reshape(1, -1))
    Aw = tf.CsrMatrix.wrap_device(Ah, dp.device_ptr(), di.device_ptr(), dx.device_ptr(), tf.pattern_hash(A))
    S2 = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128, long_row_partition=1)
    for second in (True, False, True):
        D2 = tf.DenseMatrix(M, 128); D2.fill(float("nan"))
        tf.gemm_spmm(Aw, Bd, Wd, D2, S2, second_stream=second)
        assert np.array_equal(D2.to_numpy(), want), second
    # new values in the same device array: the next call must use them, on both streams
    dx.copy_from(tf.DenseMatrix.from_numpy((A.data * np.float32(0.5)).reshape(1, -1)))
    tf.device_synchronize()
    A2 = A.copy(); A2.data = A.data * np.float32(0.5)
    D3 = tf.DenseMatrix(M, 128); D3.fill(float("nan"))
    tf.gemm_spmm(Aw, Bd, Wd, D3, S2, second_stream=True)
    want2 = tf.DenseMatrix(M, 128)
    tf.gemm_spmm(tf.CsrMatrix.from_scipy(A2), Bd, Wd, want2, S0)
    assert np.array_equal(D3.to_numpy(), want2.to_numpy())
    del Aw


def test_two_gcn_layers_in_one_call(gpu, tf, orc):
    """tf_gcn_two_layers against the oracle's executor composed twice (ReLU between, on the host), with
    and without the activation, with the hidden layer handed back, and with one schedule for both
    layers when the widths agree."""
    say("tf_gcn_two_layers")
    cfg = tf.workloads.make_config(3, 0.03)
    A = cfg["A"]
    M = A.shape[0]
    Ah = tf.CsrMatrix.from_scipy(A)
    for K, H, N in ((256, 128, 64), (64, 64, 64), (40, 96, 32)):
        X = tf.workloads.uniform((M, K), 101, 0.0, 1.0)
        W1, W2 = tf.workloads.glorot(K, H, 102), tf.workloads.glorot(H, N, 103)
        s1 = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=H, K=K)
        s2 = s1 if (K, H) == (H, N) else tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=N, K=H)
        sch = orc.unfused_schedule(M)
        h_lin, _ = orc.gemm_spmm(A, X, W1, sch, nthreads=8)
        for relu in (True, False):
            h = np.maximum(h_lin, 0.0) if relu else h_lin
            want, _ = orc.gemm_spmm(A, h, W2, sch, nthreads=8)
            D = tf.DenseMatrix(M, N); D.fill(float("nan"))
            hid = tf.DenseMatrix(M, H); hid.fill(float("nan"))
            tf.gcn_two_layers(Ah, tf.DenseMatrix.from_numpy(X), tf.DenseMatrix.from_numpy(W1), tf.DenseMatrix.from_numpy(W2), D,
                              s1, s2, relu=relu, hidden=hid)
            assert orc.rel_err(hid.to_numpy(), h) <= TOL and orc.rel_err(D.to_numpy(), want) <= TOL, (K, H, N, relu)
            D2 = tf.DenseMatrix(M, N); D2.fill(float("nan"))
            tf.gcn_two_layers(Ah, tf.DenseMatrix.from_numpy(X), tf.DenseMatrix.from_numpy(W1), tf.DenseMatrix.from_numpy(W2), D2,
                              s1, s2, relu=relu)          # hidden layer in the schedule's own buffer
            assert np.array_equal(D2.to_numpy(), D.to_numpy())
    with pytest.raises(tf.TileFusionError) as e:               # schedules in the wrong order
        tf.gcn_two_layers(Ah, tf.DenseMatrix.from_numpy(X), tf.DenseMatrix.from_numpy(W1), tf.DenseMatrix.from_numpy(W2), D, s2, s1)
    assert e.value.status == -4
    # ... which must leave no undersized hidden-layer buffer behind: the right order still works afterwards
    D3 = tf.DenseMatrix(M, N); D3.fill(float("nan"))
    tf.gcn_two_layers(Ah, tf.DenseMatrix.from_numpy(X), tf.DenseMatrix.from_numpy(W1), tf.DenseMatrix.from_numpy(W2), D3, s1, s2, relu=False)
    assert np.array_equal(D3.to_numpy(), D2.to_numpy())


def test_two_gcn_layers_hidden_width_that_needs_panels(gpu, tf, orc):
    """A hidden width the MFMA kernels do not take (30: one padded panel) on an odd row count, so that the hidden
    layer's element count is no multiple of four: the activation kernel has a tail, the layers run in panels."""
    say("tf_gcn_two_layers, H = 30")
    A = tf.workloads.erdos_renyi_gcn(3001, 8.0, seed=31)
    M = A.shape[0]
    assert (M * 30) % 4 != 0
    Ah = tf.CsrMatrix.from_scipy(A)
    K, H, N = 24, 30, 10
    X = tf.workloads.uniform((M, K), 104)
    W1, W2 = tf.workloads.glorot(K, H, 105), tf.workloads.glorot(H, N, 106)
    s1 = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=H, K=K)
    s2 = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=N, K=H)
    sch = orc.unfused_schedule(M)
    h, _ = orc.gemm_spmm(A, X, W1, sch, nthreads=8)
    h = np.maximum(h, 0.0)
    want, _ = orc.gemm_spmm(A, h, W2, sch, nthreads=8)
    D = tf.DenseMatrix(M, N); D.fill(float("nan"))
    hid = tf.DenseMatrix(M, H); hid.fill(float("nan"))
    tf.gcn_two_layers(Ah, tf.DenseMatrix.from_numpy(X), tf.DenseMatrix.from_numpy(W1), tf.DenseMatrix.from_numpy(W2), D, s1, s2,
                      relu=True, hidden=hid)
    got_h = hid.to_numpy()
    assert (got_h >= 0).all() and orc.rel_err(got_h, h) <= TOL and orc.rel_err(D.to_numpy(), want) <= TOL


def test_remainder_rows_in_list_order(gpu, tf, orc):
    """Reordered adjacency: remainder rows stored side by side in the order of the row list give the same
    bits as the same rows read from A's arrays in place, for both executors, for an uploaded matrix (values
    copied once) and after its values changed in a new upload (copied again)."""
    say("reordered adjacency for remainder rows")
    cfg = tf.workloads.make_config(3, 0.05)
    A, B, W = cfg["A"], cfg["B"], cfg["C"]
    M = A.shape[0]
    Bd, Wd = tf.DenseMatrix.from_numpy(B), tf.DenseMatrix.from_numpy(W)
    want, _ = orc.gemm_spmm(A, B, W, orc.unfused_schedule(M), nthreads=8)
    outs = []
    for ra in (0, -1):
        Ah = tf.CsrMatrix.from_scipy(A)
        S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=cfg["N"], K=cfg["K"], reorder_adjacency=ra)
        S.validate()
        assert S.info()["n_remainder_rows"] == M
        D = tf.DenseMatrix(M, cfg["N"]); D.fill(float("nan"))
        tf.gemm_spmm(Ah, Bd, Wd, D, S)
        tf.gemm_spmm(Ah, Bd, Wd, D, S)                       # second call: values already in list order
        outs.append(D.to_numpy())
        assert orc.rel_err(outs[-1], want) <= TOL
        A2 = A.copy(); A2.data = A.data * np.float32(0.5)    # same pattern, other values, new upload
        Ah2 = tf.CsrMatrix.from_scipy(A2)
        tf.gemm_spmm(Ah2, Bd, Wd, D, S)
        assert orc.rel_err(D.to_numpy(), 0.5 * want) <= TOL
    assert np.array_equal(outs[0], outs[1])
    # SpMM-SpMM on a scrambled band: nothing fuses, every row is a remainder row in length-class order
    Sm = tf.workloads.banded_random(20000, 32, 16, seed=3)
    p = np.random.default_rng(4).permutation(20000)
    Sm = sp.csr_matrix(Sm[p, :][:, p]); Sm.sort_indices()
    Sm = sp.csr_matrix((Sm.data.astype(np.float32), Sm.indices.astype(np.int32), Sm.indptr.astype(np.int32)), shape=Sm.shape)
    Cd = tf.workloads.uniform((20000, 64), 5)
    Sh = tf.CsrMatrix.from_scipy(Sm)
    got = []
    for ra in (0, -1):
        S = tf.inspector(Sh, 1, op=tf.OP_SPMM_SPMM, N=64, reorder_adjacency=ra)
        S.validate()
        D = tf.DenseMatrix(20000, 64)
        tf.spmm_spmm(Sh, Sh, tf.DenseMatrix.from_numpy(Cd), D, S)
        got.append(D.to_numpy())
    assert np.array_equal(got[0], got[1]) and np.array_equal(got[0], oracle_spmm_spmm(orc, Sm, Sm, Cd))


def test_many_rows_without_entries(gpu, tf, orc):
    """Second-op rows without entries, when they are many, are cleared by a fill kernel of their own instead of
    taking a lane group each: every such row of D is zero afterwards (D starts as NaN), rows with entries match
    the oracle bit for bit, and with accumulate the empty rows keep what D held."""
    say("many empty rows")
    rng = np.random.default_rng(21)
    M = 40000
    A = sp.random(M, M, density=6.0 / M, format="csr", random_state=21, dtype=np.float32)
    keep = rng.random(M) < 0.4                      # 60 % of the rows lose their entries
    A = sp.diags(keep.astype(np.float32)) @ A
    A.eliminate_zeros(); A.sort_indices()
    A = sp.csr_matrix((A.data.astype(np.float32), A.indices.astype(np.int32), A.indptr.astype(np.int32)), shape=A.shape)
    empty = np.diff(A.indptr) == 0
    assert empty.sum() > 20000
    Cd = tf.workloads.uniform((M, 64), 6)
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64)
    S.validate()
    assert S.info()["n_remainder_rows"] + S.info()["n_fused_rows"] == M
    D = tf.DenseMatrix(M, 64); D.fill(float("nan"))
    tf.spmm_spmm(Ah, Ah, tf.DenseMatrix.from_numpy(Cd), D, S)
    got = D.to_numpy()
    want = oracle_spmm_spmm(orc, A, A, Cd)
    assert np.array_equal(got, want) and not got[empty].any()
    D.fill(1.5)
    tf.spmm_spmm(Ah, Ah, tf.DenseMatrix.from_numpy(Cd), D, S, accumulate=True)
    acc = D.to_numpy()
    assert np.array_equal(acc[empty], np.full_like(acc[empty], 1.5))
    assert np.allclose(acc[~empty], want[~empty] + 1.5, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("N", [32, 64, 96, 128, 160, 192, 224, 256])
def test_gemm_every_output_width(gpu, tf, N):
    """tf_gemm (the row GEMM on fp32 MFMA, a lane stores N/32 consecutive columns of each of its rows) for every
    width it takes, row counts that are no multiple of the 32-row block, K that is no multiple of 8, and the same
    kernel behind a row list inside tf_gemm_spmm -- against float64, to 1e-5 / 1e-4."""
    say(f"gemm N={N}")
    rng = np.random.default_rng(3)
    for K in (8, 40, 128, 200, 256):                # 128 and 256 have kernels with K built in (N <= 128)
        for M in (1, 31, 4097, 70000):              # 70,000 rows: more than one block per wavefront
            X = rng.standard_normal((M, K)).astype(np.float32)
            W = rng.standard_normal((K, N)).astype(np.float32)
            Y = tf.DenseMatrix(M, N); Y.fill(float("nan"))
            tf.gemm(tf.DenseMatrix.from_numpy(X), tf.DenseMatrix.from_numpy(W), Y)
            want = X.astype(np.float64) @ W.astype(np.float64)
            assert np.abs(Y.to_numpy() - want).max() <= 1e-5 * max(np.abs(want).max(), 1e-30), (M, K, N)
    A = tf.workloads.make_config(3, 0.02)["A"].tolil()
    A[:, ::3] = 0                                   # a third of the intermediate rows is never read: a row list
    A = A.tocsr(); A.eliminate_zeros(); A.sort_indices()
    A = sp.csr_matrix((A.data.astype(np.float32), A.indices.astype(np.int32), A.indptr.astype(np.int32)), shape=A.shape)
    n = A.shape[0]
    Ah = tf.CsrMatrix.from_scipy(A)
    for K in (64, 128):
        B = rng.standard_normal((n, K)).astype(np.float32)
        W = rng.standard_normal((K, N)).astype(np.float32)
        S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=N, K=K)
        S.validate()
        assert 0 < S.info()["n_writeback_rows"] < n
        D = tf.DenseMatrix(n, N)
        tf.gemm_spmm(Ah, tf.DenseMatrix.from_numpy(B), tf.DenseMatrix.from_numpy(W), D, S)
        want = A.astype(np.float64) @ (B.astype(np.float64) @ W.astype(np.float64))
        assert np.abs(D.to_numpy() - want).max() <= TOL * np.abs(want).max(), (K, N)


@pytest.mark.parametrize("N", [7, 16, 48, 100, 300, 512, 700])
def test_gemm_spmm_of_any_width(gpu, tf, N):
    """geMMSpMMExecutor takes C of any width (the reference's bCols is free): widths the MFMA kernels do not
    take run as column panels.  Against float64, with K that needs padding too, with and without
    TF_ACCUMULATE, on a pattern that fuses (band) and one that does not (Erdos-Renyi)."""
    say(f"gemm_spmm N={N}")
    rng = np.random.default_rng(N)
    for A in (tf.workloads.banded_random(3000, 32, 12, seed=4), tf.workloads.make_config(3, 0.02)["A"]):
        n = A.shape[0]
        Ah = tf.CsrMatrix.from_scipy(A)
        for K in (20, 64):
            B = rng.uniform(-1, 1, (n, K)).astype(np.float32)
            W = rng.uniform(-1, 1, (K, N)).astype(np.float32)
            S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=N, K=K)
            S.validate()
            want = A.astype(np.float64) @ (B.astype(np.float64) @ W.astype(np.float64))
            D0 = rng.uniform(-1, 1, (n, N)).astype(np.float32)
            for acc in (False, True):
                D = tf.DenseMatrix.from_numpy(D0.copy())
                tf.gemm_spmm(Ah, tf.DenseMatrix.from_numpy(B), tf.DenseMatrix.from_numpy(W), D, S, accumulate=acc)
                exp = want + (D0 if acc else 0)
                assert np.abs(D.to_numpy() - exp).max() <= TOL * np.abs(exp).max(), (N, K, acc)


def test_row_gemm_of_a_schedule_repeats_bit_for_bit(gpu, tf):
    """The row GEMM behind a row list with K built in (128, 256): three calls in a row on one schedule, D
    poisoned in between and a schedule of another size used in between, give the same bits each time (a run
    with fewer than two row blocks per wavefront and one with more)."""
    say("gemm repeats")
    rng = np.random.default_rng(5)
    A = tf.workloads.make_config(3, 0.25)["A"]                 # 50,000 nodes: 1,563 row blocks, fewer than wavefronts
    A2 = tf.workloads.make_config(3, 0.6)["A"]                 # 120,000 nodes: 3,750 row blocks
    for K in (128, 256):
        runs = []
        for M_ in (A, A2):
            n = M_.shape[0]
            Ah = tf.CsrMatrix.from_scipy(M_)
            B = tf.DenseMatrix.from_numpy(rng.standard_normal((n, K)).astype(np.float32))
            W = tf.DenseMatrix.from_numpy(rng.standard_normal((K, 128)).astype(np.float32))
            S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=K)
            S.validate()
            assert S.info()["n_writeback_rows"] > 0
            want = M_.astype(np.float64) @ (B.to_numpy().astype(np.float64) @ W.to_numpy().astype(np.float64))
            runs.append((Ah, B, W, S, tf.DenseMatrix(n, 128), want))
        first = {}
        for rep in range(3):
            for i, (Ah, B, W, S, D, want) in enumerate(runs):
                D.fill(float("nan"))
                tf.gemm_spmm(Ah, B, W, D, S)
                got = D.to_numpy()
                assert np.abs(got - want).max() <= TOL * np.abs(want).max(), (K, i, rep)
                if rep == 0:
                    first[i] = got
                else:
                    assert np.array_equal(got, first[i]), (K, i, rep)


def test_device_reports_the_workgroup_to_xcd_mapping(gpu):
    """tf_device_init probes what the XCD-pinned kernels rely on: workgroup b runs on XCD b mod 8."""
    assert gpu["xcds"] == 8 and gpu["compute_units"] == 256 and gpu["wavefront"] == 64
    assert gpu["xcd_round_robin"] == 1, gpu


def test_streaming_gathers_of_short_rows_change_no_bit(gpu, tf, orc):
    """short_row_hot_bytes only changes which load instruction fetches a gathered row: a power-law product with
    the short rows' cold gathers marked (default), with a smaller hot set, and with the marks off gives the same bits."""
    say("short rows: streaming gathers")
    cfg = tf.workloads.make_config(4, 2.0 ** -5)
    A, B, W = cfg["A"], cfg["B"], cfg["C"]
    M = A.shape[0]
    Ah = tf.CsrMatrix.from_scipy(A)
    Bd, Wd = tf.DenseMatrix.from_numpy(B), tf.DenseMatrix.from_numpy(W)
    outs = []
    for hot in (0, 2 << 20, -1):
        S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128, long_row_partition=1, short_row_hot_bytes=hot)
        S.validate()
        assert (S.info()["short_row_hot_rows"] > 0) == (hot >= 0)
        D = tf.DenseMatrix(M, 128); D.fill(float("nan"))
        tf.gemm_spmm(Ah, Bd, Wd, D, S)
        outs.append(D.to_numpy())
    assert np.array_equal(outs[0], outs[2]) and np.array_equal(outs[1], outs[2])
    want, _ = orc.gemm_spmm(A, B, W, orc.unfused_schedule(M), nthreads=8)
    assert orc.rel_err(outs[0], want) <= TOL


def test_placed_intermediate_changes_no_bit(gpu, tf, orc):
    """place_intermediate only changes where the GEMM stores a row of the intermediate and what the lists call it: the
    same launches in the same order give the same bits with it and without, on a power-law graph (long rows by column
    partition, with and without the second stream) and on an Erdos-Renyi graph, and both match the oracle."""
    say("intermediate rows placed by reads")
    for cfg, kw in ((tf.workloads.make_config(4, 2.0 ** -5), dict(long_row_partition=1)), (tf.workloads.make_config(3, 0.05), dict())):
        A, B, W = cfg["A"], cfg["B"], cfg["C"]
        M, N, K = A.shape[0], cfg["N"], cfg["K"]
        Ah = tf.CsrMatrix.from_scipy(A)
        Bd, Wd = tf.DenseMatrix.from_numpy(B), tf.DenseMatrix.from_numpy(W)
        outs = []
        for place, second in ((0, False), (-1, False), (0, True)):
            S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=N, K=K, place_intermediate=place, **kw)
            S.validate()
            assert S.info()["intermediate_placed"] == (1 if place == 0 else 0)
            D = tf.DenseMatrix(M, N); D.fill(float("nan"))
            tf.gemm_spmm(Ah, Bd, Wd, D, S, second_stream=second)
            tf.gemm_spmm(Ah, Bd, Wd, D, S, second_stream=second)   # (a second call: regrouped values are reused)
            outs.append(D.to_numpy())
        assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
        want, _ = orc.gemm_spmm(A, B, W, orc.unfused_schedule(M), nthreads=8)
        assert orc.rel_err(outs[0], want) <= TOL


def test_two_host_threads_with_their_own_schedules(gpu, tf, orc):
    """Two host threads, each with its own operands, schedules and stream, call the executors at the same time (ctypes
    releases the interpreter lock during a call): every result equals the oracle's, as if each had run alone.  What the
    threads share is the library's per-process state: the loaded kernels and their attributes, the device properties."""
    import threading
    say("two host threads, own schedules and streams")
    jobs = []
    for seed, (M, N, K) in enumerate([(6000, 64, 40), (9000, 128, 128)]):
        A = tf.workloads.banded_random(M, 32, 12, seed=300 + seed)
        G = tf.workloads.erdos_renyi_gcn(M, 6.0, seed=310 + seed)
        B, W = tf.workloads.uniform((M, K), 320 + seed), tf.workloads.uniform((K, N), 330 + seed)
        Cd = tf.workloads.uniform((M, N), 340 + seed)
        jobs.append(dict(A=A, G=G, B=B, W=W, Cd=Cd, N=N, K=K, M=M,
                         want_ss=oracle_spmm_spmm(orc, A, A, Cd),
                         want_gs=orc.gemm_spmm(G, B, W, orc.unfused_schedule(M), nthreads=4)[0]))
    errors = []

    def work(job):
        try:
            M, N, K = job["M"], job["N"], job["K"]
            st = tf.Stream()
            Ah, Gh = tf.CsrMatrix.from_scipy(job["A"]), tf.CsrMatrix.from_scipy(job["G"])
            S1 = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=N, inner=Ah)
            S2 = tf.inspector(Gh, 1, op=tf.OP_GEMM_SPMM, N=N, K=K)
            S1.validate(); S2.validate()
            Cm, Bm, Wm = (tf.DenseMatrix.from_numpy(job[k]) for k in ("Cd", "B", "W"))
            D1, D2 = tf.DenseMatrix(M, N), tf.DenseMatrix(M, N)
            for _ in range(15):
                D1.fill(float("nan"), stream=st); D2.fill(float("nan"), stream=st)
                tf.spmm_spmm(Ah, Ah, Cm, D1, S1, stream=st)
                tf.gemm_spmm(Gh, Bm, Wm, D2, S2, stream=st)
                st.synchronize()
                if not np.array_equal(D1.to_numpy(), job["want_ss"]):
                    errors.append((M, "spmm_spmm differs"))
                if orc.rel_err(D2.to_numpy(), job["want_gs"]) > TOL:
                    errors.append((M, "gemm_spmm differs"))
        except Exception as e:  # noqa: BLE001  (reported by the asserting thread)
            errors.append((job["M"], repr(e)))

    threads = [threading.Thread(target=work, args=(j,)) for j in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors[:5]


def test_executors_replay_from_a_graph(gpu, tf, orc):
    """After one eager call (which allocates the schedule's workspace) an executor call is kernel launches only: it is
    captured into a HIP graph and replayed three times with other values in the dense operands, eager work and
    synchronizations in between; every replay equals the oracle (SpMM-SpMM bit for bit).  Launch-bound loops over small
    products (the 64 x 64 grid of cfg1) are what a caller would capture."""
    import ctypes as C
    say("executors under stream capture")
    with open("/proc/self/maps") as f:
        hip = C.CDLL(sorted({line.split()[-1] for line in f if "libamdhip64.so" in line})[0])
    L = tf.workloads.laplacian_2d(64)
    A = tf.workloads.banded_random(5000, 32, 12, seed=411)
    st = tf.Stream()

    def replay(call, refresh, check):
        call()                                   # eager: workspace allocated, kernels loaded
        st.synchronize()
        graph, gexec = C.c_void_p(), C.c_void_p()
        assert hip.hipStreamBeginCapture(st.h, 0) == 0
        try:
            call()
        finally:
            rc = hip.hipStreamEndCapture(st.h, C.byref(graph))
        assert rc == 0 and graph.value
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
        try:
            for i in range(3):
                refresh(i)
                st.synchronize()
                assert hip.hipGraphLaunch(gexec, st.h) == 0
                st.synchronize()
                check(i)
        finally:
            hip.hipGraphExecDestroy(gexec)
            hip.hipGraphDestroy(graph)

    # GeMM-SpMM on the 64 x 64 grid, K = N = 64 (the tile kernel with the weights in registers)
    M = L.shape[0]
    Lh = tf.CsrMatrix.from_scipy(L).to_device()
    Bs = [tf.workloads.uniform((M, 64), 420 + i) for i in range(3)]
    W = tf.workloads.uniform((64, 64), 430)
    Bm, Wm, D = tf.DenseMatrix.from_numpy(Bs[0]), tf.DenseMatrix.from_numpy(W), tf.DenseMatrix(M, 64)
    S = tf.inspector(Lh, 1, op=tf.OP_GEMM_SPMM, N=64, K=64)
    S.validate()

    def fresh_b(i):
        Bm.copy_from(tf.DenseMatrix.from_numpy(Bs[i]), stream=st)
        D.fill(float("nan"), stream=st)

    def check_gs(i):
        want, _ = orc.gemm_spmm(L, Bs[i], W, orc.unfused_schedule(M))
        assert orc.rel_err(D.to_numpy(), want) <= TOL, i
    replay(lambda: tf.gemm_spmm(Lh, Bm, Wm, D, S, stream=st), fresh_b, check_gs)

    # SpMM-SpMM on a band (windowed tiles)
    M2 = A.shape[0]
    Ah = tf.CsrMatrix.from_scipy(A).to_device()
    Cs = [tf.workloads.uniform((M2, 128), 440 + i) for i in range(3)]
    Cm, D2 = tf.DenseMatrix.from_numpy(Cs[0]), tf.DenseMatrix(M2, 128)
    S2 = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=128, inner=Ah)
    S2.validate()

    def fresh_c(i):
        Cm.copy_from(tf.DenseMatrix.from_numpy(Cs[i]), stream=st)
        D2.fill(float("nan"), stream=st)

    def check_ss(i):
        assert np.array_equal(D2.to_numpy(), oracle_spmm_spmm(orc, A, A, Cs[i])), i
    replay(lambda: tf.spmm_spmm(Ah, Ah, Cm, D2, S2, stream=st), fresh_c, check_ss)
