"""Pins the C restatement of the reference executors (oracle/tf_oracle.c).  CPU only.

Evidence used: the reference's own translation units compiled in place (bitwise), float64
scipy products, integer closed forms on Laplacians evaluated by a grid stencil that never
touches CSR code, brute-force loops on tiny inputs, and reductions to textbook routines."""
import numpy as np
import pytest
import scipy.sparse as sp


def rand_csr(M, K, density, seed):
    rng = np.random.default_rng(seed)
    m = sp.random(M, K, density=density, format="csr", random_state=rng, dtype=np.float64)
    m.data = rng.uniform(-1, 1, size=m.nnz)
    m.sort_indices()
    return m.astype(np.float32)


def stencil_2d(u):
    """(A u) for the 5-point Laplacian with zero boundary, on an (ny, nx, N) grid array."""
    out = 4.0 * u
    out[:, 1:] -= u[:, :-1]
    out[:, :-1] -= u[:, 1:]
    out[1:, :] -= u[:-1, :]
    out[:-1, :] -= u[1:, :]
    return out


def stencil_3d(u):
    out = 6.0 * u
    out[:, :, 1:] -= u[:, :, :-1]
    out[:, :, :-1] -= u[:, :, 1:]
    out[:, 1:, :] -= u[:, :-1, :]
    out[:, :-1, :] -= u[:, 1:, :]
    out[1:, :, :] -= u[:-1, :, :]
    out[:-1, :, :] -= u[1:, :, :]
    return out


def test_spmm_brute_force(orc):
    A = rand_csr(13, 9, 0.4, 1)
    X = np.random.default_rng(2).uniform(-1, 1, (9, 5)).astype(np.float32)
    want = np.zeros((13, 5), np.float32)
    for i in range(13):
        for k in range(A.indptr[i], A.indptr[i + 1]):
            for c in range(5):
                want[i, c] = np.float32(np.float64(A.data[k]) * np.float64(X[A.indices[k], c]) + np.float64(want[i, c]))
    got = orc.spmm(A, X)
    # fma(a, x, acc) in fp32 == round(a*x + acc) computed in float64 (a*x is exact in float64)
    assert np.array_equal(got, want)


def test_spmm_vs_float64(orc):
    A = rand_csr(500, 300, 0.02, 3)
    X = np.random.default_rng(4).uniform(-1, 1, (300, 48)).astype(np.float32)
    want = A.astype(np.float64) @ X.astype(np.float64)
    assert orc.rel_err(orc.spmm(A, X, nthreads=4), want) < 1e-6


@pytest.mark.parametrize("N", [32, 64, 128])
def test_spmm_spmm_bitwise_vs_reference_units(orc, tf, N):
    """The restatement and the reference's compiled scalar and AVX2 executors give the same
    bits on shared schedules (reference inspector restatement + a no-fusion schedule)."""
    if orc.ref() is None:
        pytest.skip("oracle/_ref not built on this machine")
    A = tf.workloads.banded_random(2048, 32, 16, seed=21)
    Bm = tf.workloads.banded_random(2048, 64, 9, seed=22)
    Cd = tf.workloads.uniform((2048, N), 23)
    scheds = [orc.unfused_schedule(2048), orc.inspect_vt_both_wavefronts(A, N, 100000, 2)]
    for S in scheds:
        for (a, b) in [(A, A), (A, Bm)]:
            if a is not b and S is not scheds[0]:
                continue  # an inspected schedule is only valid for the pattern it came from
            Do, To = orc.spmm_spmm(a, b, Cd, S, nthreads=2, impl="oracle")
            for impl in ("ref_scalar", "ref_vec32"):
                Dr, Tr = orc.spmm_spmm(a, b, Cd, S, nthreads=2, impl=impl)
                assert np.array_equal(To, Tr), (impl, "intermediate")
                assert np.array_equal(Do, Dr), (impl, "output")
    S = orc.inspect_fixed_tiles(A, 128, 2)
    Do, _ = orc.spmm_spmm_separated(A, Cd, S, nthreads=2, impl="oracle")
    Dr, _ = orc.spmm_spmm_separated(A, Cd, S, nthreads=2, impl="ref")
    assert np.array_equal(Do, Dr)
    Di, _ = orc.spmm_spmm(A, A, Cd, S, nthreads=2)
    assert np.array_equal(Do, Di)  # both walks of one schedule agree


def test_spmm_spmm_vs_float64_and_schedule_independence(orc, tf):
    A = tf.workloads.banded_random(1500, 32, 16, seed=5)
    Cd = tf.workloads.uniform((1500, 40), 6)
    want = A.astype(np.float64) @ (A.astype(np.float64) @ Cd.astype(np.float64))
    D0, _ = orc.spmm_spmm(A, A, Cd, orc.unfused_schedule(1500))
    D1, _ = orc.spmm_spmm(A, A, Cd, orc.inspect_vt_both_wavefronts(A, 40, 60000, 3), nthreads=3)
    assert orc.rel_err(D0, want) < 1e-6
    assert np.array_equal(D0, D1)  # per-row operation order does not depend on the schedule


def test_laplacian_all_ones_closed_form(orc, tf):
    """The reference's own SpMM-SpMM input (dense C all ones, A = B,
    fusion/example/SpMM_SpMM_Demo_Utils.h:53-59): every intermediate is a small integer, so
    fp32 is exact and D must equal the stencil applied twice, computed on the grid."""
    n, N = 24, 32
    A = tf.workloads.laplacian_2d(n)
    ones = np.ones((n * n, N), np.float32)
    D, T = orc.spmm_spmm(A, A, ones, orc.inspect_vt_both_wavefronts(A, N, 30000, 2), nthreads=2)
    u = np.ones((n, n, N))
    assert np.array_equal(T, stencil_2d(u).reshape(n * n, N).astype(np.float32))
    assert np.array_equal(D, stencil_2d(stencil_2d(u)).reshape(n * n, N).astype(np.float32))
    g = 10
    A3 = tf.workloads.laplacian_3d(g)
    ones = np.ones((g ** 3, N), np.float32)
    D, T = orc.spmm_spmm(A3, A3, ones, orc.unfused_schedule(g ** 3))
    u = np.ones((g, g, g, N))
    assert np.array_equal(D, stencil_3d(stencil_3d(u)).reshape(g ** 3, N).astype(np.float32))


def test_sgemm_integer_exact_and_orientation(orc):
    """K != N and integer operands: any transposed operand or swapped leading dimension
    changes the (exact) result."""
    rng = np.random.default_rng(7)
    X = rng.integers(-8, 9, (37, 24)).astype(np.float32)
    W = rng.integers(-8, 9, (24, 40)).astype(np.float32)
    want = (X.astype(np.int64) @ W.astype(np.int64)).astype(np.float32)
    assert np.array_equal(orc.gemm(X, W, nthreads=3), want)
    Xr = rng.uniform(-1, 1, (130, 72)).astype(np.float32)
    Wr = rng.uniform(-1, 1, (72, 33)).astype(np.float32)
    assert orc.rel_err(orc.gemm(Xr, Wr), Xr.astype(np.float64) @ Wr.astype(np.float64)) < 1e-6


def test_gemm_spmm_reductions(orc, tf):
    """A = I reduces to the GEMM, C = I to the SpMM; integer operands are exact; random
    operands agree with float64 to fp32 rounding; fused and unfused schedules agree bitwise."""
    M, K, N = 512, 24, 40
    rng = np.random.default_rng(8)
    A = tf.workloads.laplacian_2d(16, 32)
    Bi = rng.integers(-4, 5, (M, K)).astype(np.float32)
    Ci = rng.integers(-4, 5, (K, N)).astype(np.float32)
    S = orc.inspect_vt_gemm_spmm(A, K, N, 50000)
    D, T = orc.gemm_spmm(A, Bi, Ci, S, nthreads=2)
    Ti = Bi.astype(np.int64) @ Ci.astype(np.int64)
    assert np.array_equal(T, Ti.astype(np.float32))
    assert np.array_equal(D, (A.astype(np.int64) @ Ti).astype(np.float32))
    eye = sp.identity(M, format="csr", dtype=np.float32)
    D, _ = orc.gemm_spmm(eye, Bi, Ci, orc.unfused_schedule(M))
    assert np.array_equal(D, Ti.astype(np.float32))
    Br = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    D, _ = orc.gemm_spmm(A, Br, np.eye(K, dtype=np.float32), orc.unfused_schedule(M))
    assert np.array_equal(D, orc.spmm(A, Br))
    Cr = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    want = A.astype(np.float64) @ (Br.astype(np.float64) @ Cr.astype(np.float64))
    D0, _ = orc.gemm_spmm(A, Br, Cr, orc.unfused_schedule(M))
    D1, _ = orc.gemm_spmm(A, Br, Cr, S, nthreads=4)
    assert orc.rel_err(D0, want) < 1e-6
    assert np.array_equal(D0, D1)


def test_permutation_invariance(orc, tf):
    """D(P A P^T, P B) = P D(A, B): catches row/column index mix-ups."""
    M, K, N = 300, 16, 8
    rng = np.random.default_rng(9)
    A = rand_csr(M, M, 0.03, 10)
    B = rng.integers(-3, 4, (M, K)).astype(np.float32)
    Cw = rng.integers(-3, 4, (K, N)).astype(np.float32)
    A.data = rng.integers(-3, 4, A.nnz).astype(np.float32)
    perm = rng.permutation(M)
    P = sp.csr_matrix((np.ones(M, np.float32), (np.arange(M), perm)), shape=(M, M))
    Ap = sp.csr_matrix(P @ A @ P.T)
    Ap.sort_indices()
    D, _ = orc.gemm_spmm(A, B, Cw, orc.unfused_schedule(M))
    Dp, _ = orc.gemm_spmm(Ap.astype(np.float32), B[perm], Cw, orc.unfused_schedule(M))
    assert np.array_equal(Dp, D[perm])


def test_gemm_avx512_body_gives_the_scalar_bits(orc):
    """The oracle's GEMM has a register-blocked AVX-512 body (the CPU baseline's GEMM) and a scalar one;
    both add each element's products with k ascending through fused multiply-adds, so the bits must agree
    -- for whole 8 x 32 blocks, for rows and columns behind them, for K of any size, and through the fused
    executor.  Against float64 and an integer-exact product as well, so that both cannot be wrong together."""
    rng = np.random.default_rng(7)
    if not orc.simd():
        pytest.skip("this host has no AVX-512: only the scalar body runs")
    try:
        for M, K, N in ((64, 128, 128), (61, 128, 128), (203, 40, 96), (77, 256, 72), (8, 1, 32), (5, 16, 64), (129, 33, 200)):
            X = rng.uniform(-1, 1, (M, K)).astype(np.float32)
            W = rng.uniform(-1, 1, (K, N)).astype(np.float32)
            orc.set_simd(True)
            fast = orc.gemm(X, W, nthreads=3)
            orc.set_simd(False)
            slow = orc.gemm(X, W, nthreads=3)
            assert np.array_equal(fast, slow), (M, K, N)
            want = X.astype(np.float64) @ W.astype(np.float64)
            assert np.abs(fast - want).max() <= 1e-5 * max(1.0, np.abs(want).max())
        Xi = rng.integers(-3, 4, (96, 24)).astype(np.float32)
        Wi = rng.integers(-3, 4, (24, 64)).astype(np.float32)   # K != N: a transposed operand cannot pass
        orc.set_simd(True)
        assert np.array_equal(orc.gemm(Xi, Wi), (Xi.astype(np.int64) @ Wi.astype(np.int64)).astype(np.float32))
        A = sp.random(300, 300, density=0.03, random_state=5, format="csr", dtype=np.float32)
        A.sort_indices()
        B = rng.uniform(-1, 1, (300, 64)).astype(np.float32)
        Cd = rng.uniform(-1, 1, (64, 96)).astype(np.float32)
        S = orc.inspect_fixed_tiles(A, 64, 4)
        d_fast, _ = orc.gemm_spmm(A, B, Cd, S, nthreads=4)
        orc.set_simd(False)
        d_slow, _ = orc.gemm_spmm(A, B, Cd, S, nthreads=4)
        assert np.array_equal(d_fast, d_slow)
    finally:
        orc.set_simd(True)
