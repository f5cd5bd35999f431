"""Parity of the HIP executors with the CPU oracle, through the C ABI, on a real MI355X.

SpMM-SpMM is bit-exact (same fma sequence per output element as the reference's AVX2
kernels); GeMM-SpMM and split long rows are held to max|got - want| / max|want| <= 1e-4
(the fp32 MFMA GEMM and the chunked rows sum in a different order), and are exact on
integer-valued operands."""
import os
import subprocess

import numpy as np
import pytest
import scipy.sparse as sp

pytestmark = pytest.mark.gpu
TOL = 1e-4
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def say(msg):
    print(msg, flush=True)


def run_spmm_spmm(tf, A, B, Cd, accumulate=False, D0=None, **kw):
    Ah = tf.CsrMatrix.from_scipy(A)
    Bh = Ah if B is A else tf.CsrMatrix.from_scipy(B)
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=Cd.shape[1], **kw)
    S.validate()
    D = tf.DenseMatrix(A.shape[0], Cd.shape[1], D0) if D0 is not None else tf.DenseMatrix(A.shape[0], Cd.shape[1])
    if D0 is None:
        D.fill(float("nan"))  # overwrite mode must not read D
    tf.spmm_spmm(Ah, Bh, tf.DenseMatrix.from_numpy(Cd), D, S, accumulate=accumulate)
    tf.device_synchronize()
    return D.to_numpy(), S.info()


def run_gemm_spmm(tf, A, B, Cd, accumulate=False, D0=None, **kw):
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=Cd.shape[1], K=B.shape[1], **kw)
    S.validate()
    D = tf.DenseMatrix(A.shape[0], Cd.shape[1], D0) if D0 is not None else tf.DenseMatrix(A.shape[0], Cd.shape[1])
    if D0 is None:
        D.fill(float("nan"))
    tf.gemm_spmm(Ah, tf.DenseMatrix.from_numpy(B), tf.DenseMatrix.from_numpy(Cd), D, S, accumulate=accumulate)
    tf.device_synchronize()
    return D.to_numpy(), S.info()


def oracle_spmm_spmm(orc, A, B, Cd):
    return orc.spmm_spmm(A, B, Cd, orc.unfused_schedule(max(A.shape[0], B.shape[0])) if A.shape[0] == B.shape[0]
                         else _two_level(A.shape[0], B.shape[0], orc), nthreads=8)[0]


def _two_level(L, M, orc):
    ids = np.concatenate([np.arange(M), np.arange(L)]).astype(np.int32)
    typ = np.concatenate([np.zeros(M), np.ones(L)]).astype(np.int32)
    return orc.Schedule(2, [0, 1, 2], [0, M, M + L], [M, M, M, M + L], ids, typ)


# ---- SpMM-SpMM ----------------------------------------------------------------------------

@pytest.mark.parametrize("N", [128, 64, 32, 256, 8, 20, 6, 5, 320])
def test_spmm_spmm_banded_bit_exact(gpu, tf, orc, N):
    say(f"spmm_spmm banded N={N}")
    A = tf.workloads.banded_random(3000, 32, 16, seed=31)
    Cd = tf.workloads.uniform((3000, N), 32)
    want = oracle_spmm_spmm(orc, A, A, Cd)
    for kw in (dict(), dict(max_redundancy=1.0), dict(lds_budget_bytes=163840, tile_rows=200), dict(tile_rows=7)):
        got, info = run_spmm_spmm(tf, A, A, Cd, **kw)
        assert np.array_equal(got, want), (N, kw, orc.rel_err(got, want))
        if not kw:
            assert info["n_fused_rows"] == 3000


@pytest.mark.parametrize("idx,scale", [(2, 0.05), (5, 0.004), (5, 0.03)])
def test_spmm_spmm_configs_bit_exact(gpu, tf, orc, idx, scale):
    cfg = tf.workloads.make_config(idx, scale)
    say(f"spmm_spmm {cfg['name']} scale={scale} rows={cfg['A'].shape[0]}")
    want = oracle_spmm_spmm(orc, cfg["A"], cfg["A"], cfg["C"])
    got, info = run_spmm_spmm(tf, cfg["A"], cfg["A"], cfg["C"])
    assert np.array_equal(got, want)
    f64 = cfg["A"].astype(np.float64) @ (cfg["A"].astype(np.float64) @ cfg["C"].astype(np.float64))
    assert orc.rel_err(got, f64) <= TOL


def test_spmm_spmm_two_matrices_rectangular_unsorted_empty(gpu, tf, orc):
    """A != B, B rectangular, A with unsorted columns and empty rows."""
    say("spmm_spmm A != B rectangular")
    rng = np.random.default_rng(40)
    L, M, Kc, N = 900, 700, 500, 64
    A = sp.random(L, M, density=0.01, format="csr", random_state=rng, dtype=np.float32)
    A.data = rng.uniform(-1, 1, A.nnz).astype(np.float32)
    lil = A.tolil()
    for i in range(0, L, 9):
        lil.rows[i], lil.data[i] = [], []
    A = sp.csr_matrix(lil, dtype=np.float32)
    for i in range(L):  # scramble column order inside rows
        s, e = A.indptr[i], A.indptr[i + 1]
        p = rng.permutation(e - s)
        A.indices[s:e], A.data[s:e] = A.indices[s:e][p], A.data[s:e][p]
    B = sp.random(M, Kc, density=0.02, format="csr", random_state=rng, dtype=np.float32)
    B.data = rng.uniform(-1, 1, B.nnz).astype(np.float32)
    Cd = rng.uniform(-1, 1, (Kc, N)).astype(np.float32)
    want = orc.spmm_spmm(A, B, Cd, _two_level(L, M, orc))[0]
    got, _ = run_spmm_spmm(tf, A, B, Cd)
    assert np.array_equal(got, want)


def test_spmm_spmm_accumulate(gpu, tf, orc):
    say("spmm_spmm accumulate")
    A = tf.workloads.laplacian_2d(40)
    Cd = tf.workloads.uniform((1600, 64), 41)
    D0 = tf.workloads.uniform((1600, 64), 42)
    base = oracle_spmm_spmm(orc, A, A, Cd)
    for kw in (dict(), dict(max_redundancy=1.0, tile_rows=128)):
        got, _ = run_spmm_spmm(tf, A, A, Cd, accumulate=True, D0=D0, **kw)
        assert orc.rel_err(got, D0.astype(np.float64) + base) <= 1e-6
        got0, _ = run_spmm_spmm(tf, A, A, Cd, accumulate=True, D0=np.zeros_like(D0), **kw)
        assert np.array_equal(got0, base)  # zeroed D, the reference's calling convention


def test_spmm_spmm_long_rows(gpu, tf, orc):
    """Hub rows longer than long_row_nnz are cut into chunks and tree-reduced."""
    say("spmm_spmm long rows")
    rng = np.random.default_rng(43)
    M, N = 6000, 128
    A = tf.workloads.banded_random(M, 32, 16, seed=44).tolil()
    for hub, deg in ((17, 5000), (3000, 2100), (5999, 700)):
        cols = np.sort(rng.choice(M, deg, replace=False))
        A.rows[hub] = cols.tolist()
        A.data[hub] = rng.uniform(-1, 1, deg).astype(np.float32).tolist()
    A = sp.csr_matrix(A, dtype=np.float32)
    Cd = tf.workloads.uniform((M, N), 45)
    want = A.astype(np.float64) @ (A.astype(np.float64) @ Cd.astype(np.float64))
    got, info = run_spmm_spmm(tf, A, A, Cd, long_row_nnz=512)
    assert info["n_long_rows"] == 3 and info["n_long_chunks"] == 5 + 3 + 1  # chunks of 1024 entries
    assert orc.rel_err(got, want) <= TOL
    ok = np.ones(M, bool)
    ok[[17, 3000, 5999]] = False
    assert np.array_equal(got[ok], oracle_spmm_spmm(orc, A, A, Cd)[ok])  # unsplit rows stay bit-exact


def test_spmm_spmm_xcd_chunked_rows(gpu, tf, orc):
    """The row kernels under every workgroup-to-XCD mapping (round-robin, chunks of rows,
    one run per XCD): same bits as the oracle."""
    say("spmm_spmm 3D Laplacian, XCD mappings")
    g, N = 52, 64
    A = tf.workloads.laplacian_3d(g)
    Cd = tf.workloads.uniform((g ** 3, N), 46)
    want = oracle_spmm_spmm(orc, A, A, Cd)
    got, info = run_spmm_spmm(tf, A, A, Cd)
    assert info["xcd_chunk_rows"] == 0 and info["n_fused_rows"] == 0
    assert np.array_equal(got, want)
    for chunk in (-1, 64, 320, 4096):
        got, info = run_spmm_spmm(tf, A, A, Cd, xcd_chunk_rows=chunk)
        assert np.array_equal(got, want), chunk


def test_laplacian_all_ones_exact_full_size(gpu, tf):
    """The 128^3 Laplacian with an all-ones dense operand (the reference's own input,
    fusion/example/SpMM_SpMM_Demo_Utils.h:53-59): integers throughout, so D must equal the
    7-point stencil applied twice on the grid, exactly, at the benchmark's full size."""
    say("spmm_spmm 3D Laplacian 128^3 all ones")
    g, N = 128, 64
    A = tf.workloads.laplacian_3d(g)
    ones = np.ones((g ** 3, N), np.float32)
    got, info = run_spmm_spmm(tf, A, A, ones)

    def st(u):
        out = 6.0 * u
        out[:, :, 1:] -= u[:, :, :-1]; out[:, :, :-1] -= u[:, :, 1:]
        out[:, 1:, :] -= u[:, :-1, :]; out[:, :-1, :] -= u[:, 1:, :]
        out[1:, :, :] -= u[:-1, :, :]; out[:-1, :, :] -= u[1:, :, :]
        return out
    want = st(st(np.ones((g, g, g), np.float32))).reshape(-1)
    assert np.array_equal(got, np.repeat(want[:, None], N, axis=1))


def test_full_size_banded_linearity_and_roundtrip(gpu, tf, orc):
    """Benchmark size (65,536 rows, N = 128): bit-exact against the oracle, and linear in C."""
    say("spmm_spmm cfg2 full size")
    cfg = tf.workloads.make_config(2)
    A, Cd = cfg["A"], cfg["C"]
    got, info = run_spmm_spmm(tf, A, A, Cd)
    assert info["n_fused_rows"] == A.shape[0]
    want = oracle_spmm_spmm(orc, A, A, Cd)
    assert np.array_equal(got, want)
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=128, inner=Ah)  # the benchmark's schedule
    assert S.info()["windowed"] == 1
    D = tf.DenseMatrix(A.shape[0], 128)
    tf.spmm_spmm(Ah, Ah, tf.DenseMatrix.from_numpy(Cd), D, S)
    assert np.array_equal(D.to_numpy(), want)
    C2 = tf.workloads.uniform(Cd.shape, 99)
    g2, _ = run_spmm_spmm(tf, A, A, C2)
    g12, _ = run_spmm_spmm(tf, A, A, Cd + C2)
    assert orc.rel_err(g12, got.astype(np.float64) + g2) <= 1e-5


@pytest.mark.parametrize("N,strip", [(128, 32), (128, 64), (64, 32), (256, 64), (32, 32), (96, 32)])
def test_spmm_spmm_windowed_bit_exact(gpu, tf, orc, N, strip):
    """Windowed tiles (inner pattern given, B is A): CSR chunk, window of C and slab all in
    LDS, strip by strip.  Same fma order as the reference, hence the same bits."""
    say(f"spmm_spmm windowed N={N} strip={strip}")
    for A in (tf.workloads.banded_random(5000, 32, 16, seed=33), tf.workloads.laplacian_2d(40, 70)):
        M = A.shape[0]
        Cd = tf.workloads.uniform((M, N), 34)
        want = oracle_spmm_spmm(orc, A, A, Cd)
        Ah = tf.CsrMatrix.from_scipy(A)
        small = 65536 if strip == 32 else 131072
        for kw in (dict(lds_budget_bytes=0 if strip == 32 else 163840), dict(lds_budget_bytes=163840, tile_rows=200),
                   dict(tile_rows=48, lds_budget_bytes=small)):
            S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=N, inner=Ah, strip_cols=strip, **kw)
            S.validate()
            info = S.info()
            assert info["windowed"] == 1 and info["n_fused_rows"] == M and info["n_writeback_rows"] == 0
            D = tf.DenseMatrix(M, N)
            D.fill(float("nan"))
            tf.spmm_spmm(Ah, Ah, tf.DenseMatrix.from_numpy(Cd), D, S)
            tf.device_synchronize()
            assert np.array_equal(D.to_numpy(), want), (N, strip, kw)
        D0 = tf.workloads.uniform((M, N), 35)
        D = tf.DenseMatrix.from_numpy(D0)
        tf.spmm_spmm(Ah, Ah, tf.DenseMatrix.from_numpy(Cd), D, S, accumulate=True)
        assert orc.rel_err(D.to_numpy(), D0.astype(np.float64) + want) <= 1e-6


def ragged_band(M, reach, max_len, seed):
    """Rows of 0 .. max_len entries at random columns within `reach` of the diagonal; the last
    row's length is not a multiple of four."""
    rng = np.random.default_rng(seed)
    rows, cols = [], []
    for i in range(M):
        lo, hi = max(0, i - reach), min(M, i + reach + 1)
        n = int(rng.integers(0, min(max_len, hi - lo) + 1))
        if i == M - 1:
            n = 7
        if i % 97 == 5:
            n = 0
        c = rng.choice(np.arange(lo, hi), n, replace=False)
        rows += [i] * n
        cols += list(c)
    vals = rng.uniform(-1, 1, len(rows)).astype(np.float32)
    return sp.csr_matrix((vals, (rows, cols)), shape=(M, M), dtype=np.float32)


@pytest.mark.parametrize("N", [128, 64, 192, 256])
def test_spmm_spmm_wide_strips_bit_exact(gpu, tf, orc, N):
    """Long matrices get one windowed tile per compute unit, worked on in 64-column strips by
    1024 threads with the entries read from the CSR arrays in place (a lane loads four of
    every sixteen, the rest come through its quad).  Rows of 0 to 40 entries, a last row that
    ends the arrays at an odd length, D +=, and the same schedule with another B."""
    say(f"spmm_spmm wide strips N={N}")
    for A, kw in ((tf.workloads.banded_random(5000, 32, 16, seed=41), dict(compute_units=16)),
                  (ragged_band(4100, 24, 40, seed=42), dict(compute_units=16)),
                  (ragged_band(3000, 10, 13, seed=43), dict(wide_strips=1, tile_rows=100)),
                  (tf.workloads.laplacian_2d(40, 70), dict(wide_strips=1))):
        M = A.shape[0]
        Cd = tf.workloads.uniform((M, N), 44)
        want = oracle_spmm_spmm(orc, A, A, Cd)
        Ah = tf.CsrMatrix.from_scipy(A)
        S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=N, inner=Ah, **kw)
        S.validate()
        info = S.info()
        assert info["windowed"] == 1 and info["wide_strips"] == 1 and info["strip_cols"] == 64
        assert info["n_fused_rows"] == M and info["n_writeback_rows"] == 0 and info["lds_bytes"] <= 163840
        D = tf.DenseMatrix(M, N)
        D.fill(float("nan"))
        tf.spmm_spmm(Ah, Ah, tf.DenseMatrix.from_numpy(Cd), D, S)
        tf.device_synchronize()
        assert np.array_equal(D.to_numpy(), want), (N, kw)
        D0 = tf.workloads.uniform((M, N), 45)
        D = tf.DenseMatrix.from_numpy(D0)
        tf.spmm_spmm(Ah, Ah, tf.DenseMatrix.from_numpy(Cd), D, S, accumulate=True)
        assert orc.rel_err(D.to_numpy(), D0.astype(np.float64) + want) <= 1e-6
        B2 = A.copy()
        B2.data = tf.workloads.uniform((A.nnz,), 46)
        D = tf.DenseMatrix(M, N)
        tf.spmm_spmm(Ah, tf.CsrMatrix.from_scipy(B2), tf.DenseMatrix.from_numpy(Cd), D, S)
        assert np.array_equal(D.to_numpy(), oracle_spmm_spmm(orc, A, B2, Cd))


def test_spmm_spmm_windowed_schedule_with_other_inner_matrix(gpu, tf, orc):
    """A windowed schedule used with B != A falls back to the kernel that gathers C from
    HBM (same tiles), and refuses an inner matrix of another size."""
    say("spmm_spmm windowed schedule, B != A")
    A = tf.workloads.banded_random(3000, 32, 16, seed=36)
    B2 = A.copy()
    B2.data = tf.workloads.uniform((A.nnz,), 37)
    Cd = tf.workloads.uniform((3000, 64), 38)
    Ah, Bh = tf.CsrMatrix.from_scipy(A), tf.CsrMatrix.from_scipy(B2)
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Ah)
    assert S.info()["windowed"] == 1
    D = tf.DenseMatrix(3000, 64)
    tf.spmm_spmm(Ah, Bh, tf.DenseMatrix.from_numpy(Cd), D, S)
    assert np.array_equal(D.to_numpy(), oracle_spmm_spmm(orc, A, B2, Cd))
    other = tf.CsrMatrix.from_scipy(tf.workloads.banded_random(3000, 32, 8, seed=39))
    with pytest.raises(tf.TileFusionError) as e:
        tf.spmm_spmm(Ah, other, tf.DenseMatrix.from_numpy(Cd), D, S)
    assert e.value.status == -4


def test_spmm_spmm_after_rcm_reordering(gpu, tf, orc):
    """A band whose rows arrive in random order fuses nothing; after tf_reorder_rcm /
    tf_permute_csr (the reference's offline step, scripts/reorder_graphs.py:21-22) every row
    fuses, and D'[new] = D[perm[new]].  Reordering changes the order of a row's entries, so
    the comparison with the oracle on the original matrix is to 1e-5, not bit for bit."""
    say("spmm_spmm after RCM")
    M, N = 40000, 64
    A = tf.workloads.banded_random(M, 32, 16, seed=47)
    p0 = np.random.default_rng(48).permutation(M)
    S = sp.csr_matrix(A[p0, :][:, p0])
    Cd = tf.workloads.uniform((M, N), 49)
    want = oracle_spmm_spmm(orc, S, S, Cd)
    Sh = tf.CsrMatrix.from_scipy(S)
    sched = tf.inspector(Sh, 1, op=tf.OP_SPMM_SPMM, N=N, inner=Sh)
    assert sched.info()["n_fused_rows"] < 0.05 * M
    D = tf.DenseMatrix(M, N)
    tf.spmm_spmm(Sh, Sh, tf.DenseMatrix.from_numpy(Cd), D, sched)
    assert np.array_equal(D.to_numpy(), want)  # unfused, CSR order: still the reference's bits
    perm = tf.reorder_rcm(S)
    R = tf.permute_csr(S, perm)
    Rh = tf.CsrMatrix.from_scipy(R)
    sched = tf.inspector(Rh, 1, op=tf.OP_SPMM_SPMM, N=N, inner=Rh, compute_units=256)
    sched.validate()
    info = sched.info()
    assert info["n_fused_rows"] == M and info["windowed"] == 1
    D = tf.DenseMatrix(M, N)
    tf.spmm_spmm(Rh, Rh, tf.DenseMatrix.from_numpy(np.ascontiguousarray(Cd[perm])), D, sched)
    got = np.empty((M, N), np.float32)
    got[perm] = D.to_numpy()
    assert orc.rel_err(got, want) <= 1e-5


# ---- GeMM-SpMM ----------------------------------------------------------------------------

@pytest.mark.parametrize("K,N", [(64, 64), (128, 128), (256, 128), (8, 32), (72, 96), (40, 256), (512, 64)])
def test_gemm_spmm_shapes(gpu, tf, orc, K, N):
    say(f"gemm_spmm K={K} N={N}")
    n = 36
    A = tf.workloads.laplacian_2d(n)
    M = n * n
    rng = np.random.default_rng(50 + K + N)
    B = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    Cd = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    want, _ = orc.gemm_spmm(A, B, Cd, orc.unfused_schedule(M), nthreads=8)
    for kw in (dict(), dict(tile_rows=160, max_redundancy=2.0, lds_budget_bytes=163840), dict(max_redundancy=1.0, tile_rows=96)):
        got, info = run_gemm_spmm(tf, A, B, Cd, **kw)
        assert orc.rel_err(got, want) <= TOL, (K, N, kw)
    Bi = rng.integers(-4, 5, (M, K)).astype(np.float32)
    Ci = rng.integers(-4, 5, (K, N)).astype(np.float32)
    exact = (A.astype(np.int64) @ (Bi.astype(np.int64) @ Ci.astype(np.int64))).astype(np.float32)
    got, info = run_gemm_spmm(tf, A, Bi, Ci, tile_rows=160, max_redundancy=2.0, lds_budget_bytes=163840)
    assert info["n_fused_rows"] > 0
    assert np.array_equal(got, exact)  # integer operands: exact whatever the summation order


@pytest.mark.parametrize("M,K,N", [(1296, 1, 32), (1296, 20, 64), (1296, 30, 128), (1296, 129, 64), (36000, 20, 64),
                                   (36000, 100, 128)])
def test_gemm_spmm_any_k(gpu, tf, orc, M, K, N):
    """The reference's executor takes any K (fusion/gcn/GCN_Layer_MKL_Forward_Utils.h:218-291 hands
    K straight to cblas_sgemm); here a K that is not a multiple of 8 is zero-padded into the
    schedule's workspace on every call, for tiles and for streamed runs alike."""
    say(f"gemm_spmm any K M={M} K={K} N={N}")
    A = tf.workloads.banded_random(M, 32, 16, seed=80)
    rng = np.random.default_rng(81 + K)
    B = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    Cd = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    want, _ = orc.gemm_spmm(A, B, Cd, orc.unfused_schedule(M), nthreads=8)
    got, info = run_gemm_spmm(tf, A, B, Cd, compute_units=256)
    assert info["K"] == K and info["workspace_bytes"] >= (M + N) * ((K + 7) // 8 * 8) * 4
    assert info["streamed"] == (1 if M >= 32768 else 0)
    assert orc.rel_err(got, want) <= TOL
    B2 = rng.uniform(-1, 1, (M, K)).astype(np.float32)  # second call: the padding is redone, not cached
    want2, _ = orc.gemm_spmm(A, B2, Cd, orc.unfused_schedule(M), nthreads=8)
    got2, _ = run_gemm_spmm(tf, A, B2, Cd, compute_units=256)
    assert orc.rel_err(got2, want2) <= TOL


@pytest.mark.parametrize("idx,scale", [(1, 1.0), (3, 0.02), (4, 2.0 ** -6)])
def test_gemm_spmm_configs(gpu, tf, orc, idx, scale):
    cfg = tf.workloads.make_config(idx, scale)
    say(f"gemm_spmm {cfg['name']} scale={scale} rows={cfg['A'].shape[0]}")
    A = cfg["A"]
    want, _ = orc.gemm_spmm(A, cfg["B"], cfg["C"], orc.unfused_schedule(A.shape[0]), nthreads=8)
    got, info = run_gemm_spmm(tf, A, cfg["B"], cfg["C"])
    assert orc.rel_err(got, want) <= TOL
    if idx == 4:
        assert info["n_long_rows"] >= 1


@pytest.mark.parametrize("N", [128, 64, 32])
def test_long_rows_by_column_partition(gpu, tf, orc, N):
    """Power-law graph, long rows regrouped by column partition (each XCD gathers from its own
    part of the most-read intermediate rows): GeMM-SpMM and SpMM-SpMM against the oracle, and
    D +=.  A long row's segments are added in a fixed order that is not CSR order: 1e-4."""
    say(f"long rows by column partition N={N}")
    cfg = tf.workloads.make_config(4, 2.0 ** -6)
    A = cfg["A"]
    M = A.shape[0]
    rng = np.random.default_rng(90 + N)
    B = rng.uniform(-1, 1, (M, 64)).astype(np.float32)
    Cd = rng.uniform(-1, 1, (64, N)).astype(np.float32)
    want, _ = orc.gemm_spmm(A, B, Cd, orc.unfused_schedule(M), nthreads=8)
    got, info = run_gemm_spmm(tf, A, B, Cd, long_row_partition=1)
    assert info["long_row_hot_cols"] > 0 and info["n_long_rows"] > 0
    assert orc.rel_err(got, want) <= TOL
    again, _ = run_gemm_spmm(tf, A, B, Cd, long_row_partition=1)
    assert np.array_equal(got, again)  # fixed summation order
    D0 = rng.uniform(-1, 1, (M, N)).astype(np.float32)
    acc, _ = run_gemm_spmm(tf, A, B, Cd, accumulate=True, D0=D0, long_row_partition=1)
    assert orc.rel_err(acc, D0.astype(np.float64) + want) <= TOL
    C2 = rng.uniform(-1, 1, (M, N)).astype(np.float32)
    want2 = oracle_spmm_spmm(orc, A, A, C2)
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=N, long_row_partition=1)
    S.validate()
    D = tf.DenseMatrix(M, N)
    D.fill(float("nan"))
    tf.spmm_spmm(Ah, Ah, tf.DenseMatrix.from_numpy(C2), D, S)
    assert orc.rel_err(D.to_numpy(), want2) <= TOL
    first = D.to_numpy()
    # the regrouped values of an uploaded matrix are kept by the schedule: the same call again, then
    # the same schedule with another uploaded matrix of the same pattern, then the first one again
    Ah.to_device()
    for _ in range(2):
        D.fill(float("nan"))
        tf.spmm_spmm(Ah, Ah, tf.DenseMatrix.from_numpy(C2), D, S)
        assert np.array_equal(D.to_numpy(), first)
    A3 = A.copy()
    A3.data = rng.uniform(-1, 1, A.nnz).astype(np.float32)
    A3h = tf.CsrMatrix.from_scipy(A3).to_device()
    D.fill(float("nan"))
    tf.spmm_spmm(A3h, Ah, tf.DenseMatrix.from_numpy(C2), D, S)
    assert orc.rel_err(D.to_numpy(), oracle_spmm_spmm(orc, A3, A, C2)) <= TOL
    D.fill(float("nan"))
    tf.spmm_spmm(Ah, Ah, tf.DenseMatrix.from_numpy(C2), D, S)
    assert np.array_equal(D.to_numpy(), first)


def test_gemm_spmm_reductions_and_accumulate(gpu, tf, orc):
    say("gemm_spmm reductions")
    M, K, N = 1000, 64, 64
    rng = np.random.default_rng(60)
    B = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    Cd = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    eye = sp.identity(M, format="csr", dtype=np.float32)
    got, info = run_gemm_spmm(tf, eye, B, Cd)  # A = I: D = B*C, every row fused
    assert info["n_fused_rows"] == M
    assert orc.rel_err(got, B.astype(np.float64) @ Cd.astype(np.float64)) <= 1e-6
    A = tf.workloads.banded_random(M, 32, 16, seed=61)
    got, _ = run_gemm_spmm(tf, A, B, np.eye(K, dtype=np.float32))  # C = I: D = A*B exactly
    assert np.array_equal(got, orc.spmm(A, B))
    D0 = rng.uniform(-1, 1, (M, N)).astype(np.float32)
    base, _ = run_gemm_spmm(tf, A, B, Cd)
    acc, _ = run_gemm_spmm(tf, A, B, Cd, accumulate=True, D0=D0)
    assert orc.rel_err(acc, D0.astype(np.float64) + base) <= 1e-6


@pytest.mark.parametrize("K,N", [(128, 128), (64, 128), (256, 128), (8, 96), (256, 64), (64, 64), (32, 32)])
def test_gemm_spmm_streamed(gpu, tf, orc, K, N):
    """Long matrices take the streamed kernel: every banded row fused out of the LDS ring; rows
    with more than 32 entries or a far column go through the remainder and read the rows the
    runs write back; D += is a separate instantiation."""
    say(f"gemm_spmm streamed K={K} N={N}")
    M = 36000
    A0 = tf.workloads.banded_random(M, 32, 16, seed=70)
    rng = np.random.default_rng(71 + K + N)
    B = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    Cd = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    want, _ = orc.gemm_spmm(A0, B, Cd, orc.unfused_schedule(M), nthreads=8)
    got, info = run_gemm_spmm(tf, A0, B, Cd, compute_units=256)
    assert info["streamed"] == 1 and info["n_fused_rows"] == M and info["n_writeback_rows"] == 0
    assert orc.rel_err(got, want) <= TOL
    lil = A0.tolil()
    for i in rng.choice(M, 40, replace=False):
        lo = max(0, i - 30)
        lil[i, lo:lo + 40] = 0.5
    for i in rng.choice(M, 40, replace=False):
        lil[i, (i + M // 3) % M] = -2.0
    lil[M // 2] = 0  # an empty row
    A = sp.csr_matrix(lil, dtype=np.float32)
    A.eliminate_zeros()
    want, _ = orc.gemm_spmm(A, B, Cd, orc.unfused_schedule(M), nthreads=8)
    got, info = run_gemm_spmm(tf, A, B, Cd, compute_units=256)
    assert info["streamed"] == 1 and 0 < info["n_remainder_rows"] <= 81 and info["n_writeback_rows"] > 0
    assert orc.rel_err(got, want) <= TOL
    D0 = rng.uniform(-1, 1, (M, N)).astype(np.float32)
    acc, _ = run_gemm_spmm(tf, A, B, Cd, accumulate=True, D0=D0, compute_units=256)
    assert orc.rel_err(acc, D0.astype(np.float64) + want) <= TOL
    Bi = rng.integers(-3, 4, (M, K)).astype(np.float32)
    Ci = rng.integers(-3, 4, (K, N)).astype(np.float32)
    Ai = A0.copy()
    Ai.data = rng.integers(-2, 3, Ai.nnz).astype(np.float32)
    exact = (Ai.astype(np.int64) @ (Bi.astype(np.int64) @ Ci.astype(np.int64))).astype(np.float32)
    got, _ = run_gemm_spmm(tf, Ai, Bi, Ci, compute_units=256)
    assert np.array_equal(got, exact)  # integer operands: exact whatever the summation order


def test_power_law_row_sums_full_size(gpu, tf):
    """2^21-node R-MAT, row-normalised: with all-ones B (M x 128) and C (128 x 128) the
    intermediate is 128 everywhere, so D is 128 on every non-empty row and 0 on empty ones."""
    say("gemm_spmm R-MAT 2^21 all ones")
    cfg = tf.workloads.make_config(4)
    A = cfg["A"]
    M = A.shape[0]
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128)
    S.validate()
    B = tf.DenseMatrix(M, 128); B.fill(1.0)
    Cm = tf.DenseMatrix(128, 128); Cm.fill(1.0)
    D = tf.DenseMatrix(M, 128); D.fill(float("nan"))
    tf.gemm_spmm(Ah, B, Cm, D, S)
    tf.device_synchronize()
    got = D.to_numpy()
    empty = np.diff(A.indptr) == 0
    assert np.all(got[empty] == 0.0)
    rs = np.asarray(A.astype(np.float64).sum(axis=1)).ravel()
    assert np.abs(got[~empty] - 128.0 * rs[~empty][:, None]).max() <= 128.0 * TOL
    assert np.abs(got[~empty] - 128.0).max() <= 128.0 * TOL


# ---- building blocks, the C++ API, error behaviour ---------------------------------------

def test_unfused_building_blocks(gpu, tf, orc):
    say("tf_spmm / tf_gemm")
    A = tf.workloads.banded_random(2000, 64, 9, seed=70)
    X = tf.workloads.uniform((2000, 96), 71)
    Y = tf.DenseMatrix(2000, 96)
    tf.spmm(tf.CsrMatrix.from_scipy(A), tf.DenseMatrix.from_numpy(X), Y)
    assert np.array_equal(Y.to_numpy(), orc.spmm(A, X))
    W = tf.workloads.uniform((96, 64), 72)
    Z = tf.DenseMatrix(2000, 64)
    tf.gemm(tf.DenseMatrix.from_numpy(X), tf.DenseMatrix.from_numpy(W), Z)
    assert orc.rel_err(Z.to_numpy(), X.astype(np.float64) @ W.astype(np.float64)) <= 1e-6
    # shapes the MFMA kernel does not take (the reference's sgemm takes any): padded / cut into panels inside the call
    for (M, K, N) in ((700, 20, 50), (33, 7, 1), (1500, 64, 300), (257, 100, 600)):
        Xq, Wq = tf.workloads.uniform((M, K), 73 + N), tf.workloads.uniform((K, N), 74 + N)
        Zq = tf.DenseMatrix(M, N); Zq.fill(float("nan"))
        tf.gemm(tf.DenseMatrix.from_numpy(Xq), tf.DenseMatrix.from_numpy(Wq), Zq)
        assert orc.rel_err(Zq.to_numpy(), Xq.astype(np.float64) @ Wq.astype(np.float64)) <= 1e-6, (M, K, N)


@pytest.mark.parametrize("N", [32, 64, 128, 256, 20, 320])
def test_spmm_long_row_lists_bit_exact(gpu, tf, orc, N):
    """Row lists of 4096 rows and more take the kernel that stages row pointers and entries ahead:
    rows with 0, a few, exactly 16, and more than 16 entries, unsorted columns, accumulate."""
    say(f"tf_spmm staged N={N}")
    M = 9000
    rng = np.random.default_rng(80 + N)
    lens = rng.choice([0, 1, 3, 7, 8, 9, 15, 16, 17, 24, 31, 32], size=M)
    lens[-1] = 5
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    indices = np.concatenate([rng.choice(M, l, replace=False) for l in lens]).astype(np.int32)
    data = rng.uniform(-1, 1, indptr[-1]).astype(np.float32)
    A = sp.csr_matrix((data, indices, indptr), shape=(M, M))
    X = rng.uniform(-1, 1, (M, N)).astype(np.float32)
    Ah = tf.CsrMatrix.from_scipy(A)
    Y = tf.DenseMatrix(M, N)
    Y.fill(float("nan"))
    tf.spmm(Ah, tf.DenseMatrix.from_numpy(X), Y)
    want = orc.spmm(A, X)
    assert np.array_equal(Y.to_numpy(), want)
    Y0 = rng.uniform(-1, 1, (M, N)).astype(np.float32)
    Y = tf.DenseMatrix(M, N, Y0)
    tf.spmm(Ah, tf.DenseMatrix.from_numpy(X), Y, accumulate=True)
    got = Y.to_numpy()
    ref = Y0.copy()
    for i in range(0, M, 97):  # accumulate continues the fma chain from the old value
        acc = Y0[i].copy()
        for k in range(indptr[i], indptr[i + 1]):
            acc = (np.float64(data[k]) * X[indices[k]].astype(np.float64) + acc).astype(np.float32)
        ref[i] = acc
    assert np.array_equal(got[::97], ref[::97])


def test_cpp_readme_api(gpu):
    say("C++ README API program")
    exe = os.path.join(ROOT, "tests", "cpp", "api_check")
    assert os.path.exists(exe), "tests/cpp/api_check is not built (run build())"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "api_check ok" in r.stdout, r.stdout + r.stderr


def test_error_behaviour(gpu, tf):
    say("error paths")
    A = tf.workloads.banded_random(512, 32, 16, seed=80)
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64)
    Cd = tf.DenseMatrix(512, 64); Cd.fill(1.0)
    D = tf.DenseMatrix(512, 64)
    with pytest.raises(tf.TileFusionError) as e:  # schedule built for another N
        tf.spmm_spmm(Ah, Ah, tf.DenseMatrix(512, 32), tf.DenseMatrix(512, 32), S)
    assert e.value.status == -4
    with pytest.raises(tf.TileFusionError) as e:  # schedule built for the other operation
        tf.gemm_spmm(Ah, Cd, tf.DenseMatrix(64, 64), D, S)
    assert e.value.status == -4
    other = tf.CsrMatrix.from_scipy(tf.workloads.laplacian_2d(16))
    with pytest.raises(tf.TileFusionError) as e:  # schedule built for another pattern
        tf.spmm_spmm(other, other, tf.DenseMatrix(256, 64), tf.DenseMatrix(256, 64), S)
    assert e.value.status == -4
    with pytest.raises(tf.TileFusionError) as e:  # D with the wrong row count
        tf.spmm_spmm(Ah, Ah, Cd, tf.DenseMatrix(100, 64), S)
    assert e.value.status == -1
    tf.spmm_spmm(Ah, Ah, Cd, D, S)  # and the handle is still usable afterwards
    tf.device_synchronize()
    assert np.isfinite(D.to_numpy()).all()


def test_streams_and_wrapped_buffers(gpu, tf, orc):
    """A caller-provided stream and a dense operand wrapped around foreign device memory."""
    say("streams / wrapped device pointers")
    A = tf.workloads.banded_random(1024, 32, 16, seed=81)
    Cd = tf.workloads.uniform((1024, 128), 82)
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=128)
    owner = tf.DenseMatrix(1024, 128)
    D = tf.DenseMatrix.wrap_device(1024, 128, owner.device_ptr())
    st = tf.Stream()
    e0, e1 = tf.Event(), tf.Event()
    e0.record(st)
    tf.spmm_spmm(Ah, Ah, tf.DenseMatrix.from_numpy(Cd), D, S, stream=st)
    e1.record(st)
    e1.synchronize()
    assert e0.elapsed_ms(e1) > 0.0
    assert np.array_equal(owner.to_numpy(), oracle_spmm_spmm(orc, A, A, Cd))
