"""A seeded sweep of random patterns, widths and inspector options through the C ABI against the oracle.

Every schedule is validated before it runs.  SpMM-SpMM results are compared bit for bit (to 1e-4 where long rows are
summed in pieces or D is accumulated into), GeMM-SpMM and the two-layer forward to 1e-4 of the largest element.
Every case is printed before it runs, so a failure names its pattern, widths and options."""
import numpy as np
import pytest
import scipy.sparse as sp

pytestmark = pytest.mark.gpu
TOL = 1e-4
CASES_PER_SEED = 70
EINVAL, EUNSUPPORTED = -1, -5   # tf_status values of include/tilefusion_hip.h


def csr32(m):
    m = sp.csr_matrix(m, dtype=np.float32)
    m.sort_indices()
    m.indptr = m.indptr.astype(np.int32)
    m.indices = m.indices.astype(np.int32)
    return m


def random_pattern(wl, rng):
    """One of: random band, Erdos-Renyi, R-MAT, 2D / 3D stencil (5, 7, 19, 27 points), a few hub rows over a sparse background, a band with
    a third of its rows emptied, a band off the diagonal, diagonal blocks.  Values uniform in [-1, 1]."""
    seed = int(rng.integers(1 << 30))
    kind = str(rng.choice(["band", "band", "er", "rmat", "lap2", "lap3", "box3", "hub", "empty", "bandoff", "block"]))
    if kind == "band":
        bw = int(rng.choice([2, 4, 16, 32, 64, 100]))
        A = wl.banded_random(int(rng.integers(40, 6000)), bw, int(rng.integers(1, min(bw // 2, 24) + 1)), seed=seed)
    elif kind == "er":
        A = wl.erdos_renyi_gcn(int(rng.integers(30, 5000)), float(rng.uniform(1, 14)), seed=seed)
    elif kind == "rmat":
        s = int(rng.integers(8, 13))
        A = wl.rmat(s, (1 << s) * int(rng.integers(2, 12)), seed=seed)
    elif kind == "lap2":
        A = wl.laplacian_2d(int(rng.integers(4, 70)), int(rng.integers(4, 70)))
    elif kind == "lap3":
        A = wl.laplacian_3d(int(rng.integers(3, 18)))
    elif kind == "box3":   # 27 points, or 19 without the corners of the cube
        def line(n, centre=True):
            e = np.ones(n)
            return sp.diags([e[:-1], e, e[:-1]], [-1, 0, 1]) if centre else sp.diags([e[:-1], e[:-1]], [-1, 1])
        nx, ny, nz = (int(v) for v in rng.integers(3, 15, size=3))
        A = sp.csr_matrix(sp.kron(sp.kron(line(nz), line(ny)), line(nx)))
        if rng.random() < 0.5:
            A = A - sp.csr_matrix(sp.kron(sp.kron(line(nz, False), line(ny, False)), line(nx, False)))
            A.eliminate_zeros()
    elif kind == "hub":
        M = int(rng.integers(200, 4000))
        A = sp.random(M, M, density=4.0 / M, random_state=seed, format="lil")
        for r in rng.integers(0, M, size=int(rng.integers(1, 6))):
            A[int(r), rng.choice(M, size=int(rng.integers(40, min(M, 1500))), replace=False)] = 1.0
    elif kind == "empty":
        M = int(rng.integers(50, 3000))
        A = wl.banded_random(M, 16, 6, seed=seed).tolil()
        for r in rng.integers(0, M, size=M // 3):
            A.rows[int(r)], A.data[int(r)] = [], []
    elif kind == "bandoff":
        M = int(rng.integers(300, 5000))
        off = int(rng.integers(-200, 200))
        diags = [off + d for d in range(-int(rng.integers(1, 12)), int(rng.integers(1, 12)))]
        A = sp.diags([np.ones(M - abs(d)) for d in diags], diags, shape=(M, M), format="csr")
    else:
        bs = int(rng.integers(4, 60))
        A = sp.block_diag([sp.random(bs, bs, density=0.3, random_state=seed + i) for i in range(int(rng.integers(2, 30)))],
                          format="csr")
    A = csr32(A)
    if A.nnz == 0:
        A = csr32(sp.eye(A.shape[0]))
    A.data = rng.uniform(-1.0, 1.0, A.nnz).astype(np.float32)
    return kind, A


def random_opts(tf, rng, op):
    choices = dict(max_redundancy=[0.1, 0.5, 1.0, 3.0], tile_rows=[3, 7, 16, 50, 200, 1000],
                   lds_budget_bytes=[16384, 65536, 163840], long_row_nnz=[8, 16, 64, 200], long_row_partition=[-1, 1],
                   hot_partition_bytes=[4096, 65536, 1 << 20], short_row_hot_bytes=[-1, 2048, 65536, 1 << 20],
                   compute_units=[1, 8, 64, 256, 1000], xcd_chunk_rows=[-1, 64, 1024], wide_strips=[-1, 1],
                   strip_cols=[32, 64], reorder_adjacency=[-1, 1], march=[-1, 1])
    if op == tf.OP_GEMM_SPMM:
        choices["two_layer_tiles"] = [-1, 1]
    kw = {}
    for name, values in choices.items():
        if rng.random() < 0.25:
            v = rng.choice(values)
            kw[name] = float(v) if name == "max_redundancy" else int(v)
    return kw


def inspect_or_none(tf, Ah, op, N, K, kw, inner=None):
    """The schedule, validated -- or None where the inspector refuses the options (an LDS budget too small for a
    tile, marching asked for on a pattern without a grid)."""
    try:
        S = tf.inspector(Ah, 1, op=op, N=N, K=K, inner=inner, **kw)
    except tf.TileFusionError as e:
        assert e.status in (EINVAL, EUNSUPPORTED), e
        print("   inspector declined:", e.status, flush=True)
        return None
    S.validate()
    return S


def worst(got, want):
    return float(np.max(np.abs(got - want)) / max(1e-30, np.max(np.abs(want))))


def spmm_spmm_case(tf, orc, rng, tag, A, noalloc):
    wl, M = tf.workloads, A.shape[0]
    Ah = tf.CsrMatrix.from_scipy(A)
    N = int(rng.choice([1, 4, 5, 8, 20, 32, 48, 64, 96, 128, 192, 256, 320]))
    acc = bool(rng.random() < 0.2)
    kw = {} if noalloc else random_opts(tf, rng, tf.OP_SPMM_SPMM)
    print(f"{tag} {'noalloc' if noalloc else 'spmm_spmm'} M={M} nnz={A.nnz} N={N} acc={acc} {kw}", flush=True)
    Cd = wl.uniform((M, N), int(rng.integers(1 << 30)))
    D0 = wl.uniform((M, N), int(rng.integers(1 << 30))) if acc else None
    D = tf.DenseMatrix(M, N, D0)
    if not acc:
        D.fill(float("nan"))
    exact = not acc
    if noalloc:
        Ah.to_device()
        try:
            tf.spmm_spmm_noalloc(Ah, Ah, tf.DenseMatrix.from_numpy(Cd), D, accumulate=acc)
        except tf.TileFusionError as e:
            assert e.status == EUNSUPPORTED, e   # the intermediate is larger than the scratch array
            return True
    else:
        S = inspect_or_none(tf, Ah, tf.OP_SPMM_SPMM, N, 0, kw, inner=Ah if rng.random() < 0.8 else None)
        if S is None:
            return True
        tf.spmm_spmm(Ah, Ah, tf.DenseMatrix.from_numpy(Cd), D, S, accumulate=acc)
        exact = exact and S.info()["n_long_rows"] == 0
    tf.device_synchronize()
    got = D.to_numpy()
    want = orc.spmm_spmm(A, A, Cd, orc.unfused_schedule(M), nthreads=8)[0]
    if exact:
        return np.array_equal(got, want)
    want = want.astype(np.float64) + (D0 if acc else 0.0)
    return worst(got, want) <= TOL


def gemm_spmm_case(tf, orc, rng, tag, A, partition):
    wl, M = tf.workloads, A.shape[0]
    N = int(rng.choice([1, 5, 8, 30, 32, 64, 100, 128, 256, 300]))
    K = int(rng.choice([1, 3, 16, 32, 40, 64, 128, 200, 256]))
    acc = bool(rng.random() < 0.2)
    kw = random_opts(tf, rng, tf.OP_GEMM_SPMM)
    print(f"{tag} gemm_spmm{' after partition ordering' if partition else ''} M={M} nnz={A.nnz} K={K} N={N} acc={acc} {kw}",
          flush=True)
    if partition:
        perm, _ = tf.reorder_partition(A, int(rng.choice([2, 8, 32])), int(rng.choice([0, 4, 50])))
        assert np.array_equal(np.sort(perm), np.arange(M))
        A = tf.permute_csr(A, perm)
    Ah = tf.CsrMatrix.from_scipy(A)
    B, W = wl.uniform((M, K), int(rng.integers(1 << 30))), wl.uniform((K, N), int(rng.integers(1 << 30)))
    D0 = wl.uniform((M, N), int(rng.integers(1 << 30))) if acc else None
    S = inspect_or_none(tf, Ah, tf.OP_GEMM_SPMM, N, K, kw)
    if S is None:
        return True
    D = tf.DenseMatrix(M, N, D0)
    if not acc:
        D.fill(float("nan"))
    tf.gemm_spmm(Ah, tf.DenseMatrix.from_numpy(B), tf.DenseMatrix.from_numpy(W), D, S, accumulate=acc,
                 second_stream=bool(rng.random() < 0.2))
    tf.device_synchronize()
    want = orc.gemm_spmm(A, B, W, orc.unfused_schedule(M), nthreads=8)[0].astype(np.float64) + (D0 if acc else 0.0)
    return worst(D.to_numpy(), want) <= TOL


def two_layer_case(tf, orc, rng, tag, A):
    wl, M = tf.workloads, A.shape[0]
    Ah = tf.CsrMatrix.from_scipy(A)
    K, H, N = int(rng.choice([8, 30, 32, 64, 128, 200])), int(rng.choice([16, 30, 32, 64, 128])), int(rng.choice([7, 32, 64, 128]))
    relu, acc = bool(rng.random() < 0.8), bool(rng.random() < 0.2)
    kw1, kw2 = random_opts(tf, rng, tf.OP_GEMM_SPMM), random_opts(tf, rng, tf.OP_GEMM_SPMM)
    print(f"{tag} two layers M={M} nnz={A.nnz} K={K} H={H} N={N} relu={relu} acc={acc} {kw1} {kw2}", flush=True)
    X, W1, W2 = (wl.uniform(shape, int(rng.integers(1 << 30))) for shape in ((M, K), (K, H), (H, N)))
    s1 = inspect_or_none(tf, Ah, tf.OP_GEMM_SPMM, H, K, kw1)
    s2 = inspect_or_none(tf, Ah, tf.OP_GEMM_SPMM, N, H, kw2)
    if s1 is None or s2 is None:
        return True
    D0 = wl.uniform((M, N), int(rng.integers(1 << 30))) if acc else None
    hidden = orc.gemm_spmm(A, X, W1, orc.unfused_schedule(M), nthreads=8)[0]
    if relu:
        hidden = np.maximum(hidden, 0.0)
    want = orc.gemm_spmm(A, hidden, W2, orc.unfused_schedule(M), nthreads=8)[0].astype(np.float64) + (D0 if acc else 0.0)
    ok = True
    for fuse in (False, True):
        if fuse and (s2.info()["two_layer_tiles"] == 0 or K % 8 != 0):
            continue   # (the tiles exist for banded patterns and widths of 32, 64, 128 only)
        D = tf.DenseMatrix(M, N, D0)
        if not acc:
            D.fill(float("nan"))
        tf.gcn_two_layers(Ah, tf.DenseMatrix.from_numpy(X), tf.DenseMatrix.from_numpy(W1), tf.DenseMatrix.from_numpy(W2),
                          D, s1, s2, relu=relu, accumulate=acc, fuse=fuse)
        tf.device_synchronize()
        ok = ok and worst(D.to_numpy(), want) <= TOL
    return ok


@pytest.mark.parametrize("seed", [101, 102, 103])
def test_random_sweep(gpu, tf, orc, seed):
    rng = np.random.default_rng(seed)
    failed = []
    for case in range(CASES_PER_SEED):
        what = str(rng.choice(["spmm_spmm", "spmm_spmm", "gemm_spmm", "gemm_spmm", "two_layers", "noalloc", "partition"]))
        kind, A = random_pattern(tf.workloads, rng)
        tag = f"case {seed}.{case} [{kind}]"
        if what in ("spmm_spmm", "noalloc"):
            ok = spmm_spmm_case(tf, orc, rng, tag, A, noalloc=what == "noalloc")
        elif what in ("gemm_spmm", "partition"):
            ok = gemm_spmm_case(tf, orc, rng, tag, A, partition=what == "partition")
        else:
            ok = two_layer_case(tf, orc, rng, tag, A)
        if not ok:
            failed.append(tag)
    assert not failed, failed
