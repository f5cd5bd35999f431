"""Seeded synthetic operands for the five benchmark configurations.

All sparse matrices are scipy CSR with int32 indices, sorted columns and fp32 values;
dense matrices are row-major fp32.  ``scale`` < 1 shrinks a configuration for tests.
"""
import numpy as np
import scipy.sparse as sp


def _csr32(m):
    m = sp.csr_matrix(m)
    m.sum_duplicates()
    m.sort_indices()
    m.indptr = m.indptr.astype(np.int32)
    m.indices = m.indices.astype(np.int32)
    m.data = m.data.astype(np.float32)
    return m


def uniform(shape, seed, lo=-1.0, hi=1.0):
    return np.random.default_rng(seed).uniform(lo, hi, size=shape).astype(np.float32)


def laplacian_2d(nx, ny=None):
    """5-point Laplacian on an nx x ny grid, natural row-major ordering: 4 / -1."""
    ny = ny or nx
    ex, ey = np.ones(nx), np.ones(ny)
    tx = sp.diags([-ex[:-1], 2 * ex, -ex[:-1]], [-1, 0, 1])
    ty = sp.diags([-ey[:-1], 2 * ey, -ey[:-1]], [-1, 0, 1])
    m = sp.csr_matrix(sp.kron(sp.identity(ny), tx) + sp.kron(ty, sp.identity(nx)))
    m.eliminate_zeros()  # (kron stores small dense factors as blocks, zeros included)
    return _csr32(m)


def laplacian_3d(n):
    """7-point Laplacian on an n^3 grid, x fastest: 6 / -1."""
    e = np.ones(n)
    t = sp.diags([-e[:-1], 2 * e, -e[:-1]], [-1, 0, 1])
    i = sp.identity(n)
    m = sp.csr_matrix(sp.kron(sp.kron(i, i), t) + sp.kron(sp.kron(i, t), i) + sp.kron(sp.kron(t, i), i))
    m.eliminate_zeros()
    return _csr32(m)


def box_stencil_3d(n, corners=True):
    """The stencil of all neighbours within one step in every direction on an n^3 grid, x fastest: 27 points (19
    without the cube's corners), every row scaled to sum 1."""
    e = np.ones(n)
    t = sp.diags([e[:-1], e, e[:-1]], [-1, 0, 1])
    m = sp.csr_matrix(sp.kron(sp.kron(t, t), t))
    if not corners:
        o = sp.diags([e[:-1], e[:-1]], [-1, 1])
        m = sp.csr_matrix(m - sp.kron(sp.kron(o, o), o))
        m.eliminate_zeros()
    deg = np.asarray(m.sum(axis=1)).ravel()
    return _csr32(sp.diags(1.0 / deg) @ m)


def banded_random(M, bandwidth=32, per_row=16, seed=3):
    """Each row holds `per_row` distinct columns drawn uniformly from
    [i - bandwidth/2, i + bandwidth/2) clipped to [0, M), values uniform[-1, 1]."""
    rng = np.random.default_rng(seed)
    half = bandwidth // 2
    keys = rng.random((M, bandwidth))
    cols = np.arange(M)[:, None] + np.arange(-half, half)[None, :]
    keys[(cols < 0) | (cols >= M)] = np.inf
    pick = np.argsort(keys, axis=1)[:, :per_row]
    c = np.take_along_axis(cols, pick, axis=1)
    r = np.repeat(np.arange(M), per_row)
    v = rng.uniform(-1.0, 1.0, size=M * per_row)
    return _csr32(sp.coo_matrix((v, (r, c.ravel())), shape=(M, M)))


def gcn_normalise(adj):
    """x_ij / sqrt(deg_i * deg_j) with deg = stored entries per row, self-loops already in
    (the reference's normalizeAdjacencyMatrix, GCN_Single_Layer_SP_Demo_Utils.h:40-53)."""
    adj = sp.csr_matrix(adj, dtype=np.float64)
    deg = np.diff(adj.indptr).astype(np.float64)
    d = 1.0 / np.sqrt(np.maximum(deg, 1.0))
    return _csr32(sp.diags(d) @ adj @ sp.diags(d))


def erdos_renyi_gcn(n, mean_degree=10.0, seed=5):
    """Symmetric-normalised adjacency with self-loops of an undirected G(n, p) graph."""
    rng = np.random.default_rng(seed)
    m = rng.binomial(n * (n - 1) // 2, mean_degree / (n - 1))
    u = rng.integers(0, n, size=int(m * 1.02) + 16)
    v = rng.integers(0, n, size=u.size)
    keep = u != v
    u, v = u[keep][:m], v[keep][:m]
    a = sp.coo_matrix((np.ones(u.size), (u, v)), shape=(n, n))
    a = a + a.T + sp.identity(n)
    a.data[:] = 1.0
    a = sp.csr_matrix(a)
    a.data[:] = 1.0
    return gcn_normalise(a)


def rmat(scale, n_edges, abcd=(0.57, 0.19, 0.19, 0.05), seed=8):
    """R-MAT graph on 2^scale nodes, symmetrised, deduplicated, row-normalised."""
    rng = np.random.default_rng(seed)
    a, b, c, _ = abcd
    rows = np.zeros(n_edges, dtype=np.int64)
    cols = np.zeros(n_edges, dtype=np.int64)
    for _bit in range(scale):
        r = rng.random(n_edges)
        down = r >= a + b            # quadrants c, d: row bit set
        right = ((r >= a) & (r < a + b)) | (r >= a + b + c)  # quadrants b, d: column bit set
        rows = (rows << 1) | down
        cols = (cols << 1) | right
    n = 1 << scale
    m = sp.coo_matrix((np.ones(n_edges), (rows, cols)), shape=(n, n))
    m = sp.csr_matrix(m + m.T)
    m.data[:] = 1.0
    deg = np.asarray(m.sum(axis=1)).ravel()
    inv = np.where(deg > 0, 1.0 / np.maximum(deg, 1.0), 0.0)
    return _csr32(sp.diags(inv) @ m)


def glorot(K, N, seed):
    lim = float(np.sqrt(6.0 / (K + N)))
    return uniform((K, N), seed, -lim, lim)


CONFIG_NAMES = {
    1: "cfg1 GeMM-SpMM 2D Laplacian 64x64, K=N=64",
    2: "cfg2 SpMM-SpMM banded bw32 65536 rows, N=128",
    3: "cfg3 GeMM-SpMM GCN layer, Erdos-Renyi 200k nodes deg 10, K=256 N=128",
    4: "cfg4 GeMM-SpMM R-MAT 2^21 nodes, K=N=128",
    5: "cfg5 SpMM-SpMM 3D Laplacian 128^3, N=64",
    # not one of the reference's configurations: the banded pattern of cfg2 under GeMM-SpMM, the
    # workload on which the fused GeMM-SpMM kernel has rows to fuse at full size
    6: "extra GeMM-SpMM banded bw32 262144 rows, K=N=128",
    # ... and a stencil with diagonal neighbours: rows of 27 entries, the wide form of the marching runs
    7: "extra SpMM-SpMM 27-point stencil 128^3, N=64",
}


def make_config(idx, scale=1.0):
    """Returns a dict: op ('gemm_spmm' | 'spmm_spmm'), A (scipy CSR), B (scipy CSR or dense),
    C (dense), K, N, name.  `scale` shrinks the row count (tests)."""
    if idx == 1:
        g = max(8, int(round(64 * np.sqrt(scale))))
        A = laplacian_2d(g)
        M = A.shape[0]
        return dict(op="gemm_spmm", A=A, B=uniform((M, 64), 1), C=uniform((64, 64), 2), K=64, N=64, name=CONFIG_NAMES[1])
    if idx == 2:
        M = max(256, int(65536 * scale))
        A = banded_random(M, 32, 16, seed=3)
        return dict(op="spmm_spmm", A=A, B=A, C=uniform((M, 128), 4), K=0, N=128, name=CONFIG_NAMES[2])
    if idx == 3:
        n = max(512, int(200000 * scale))
        A = erdos_renyi_gcn(n, 10.0, seed=5)
        return dict(op="gemm_spmm", A=A, B=uniform((n, 256), 6, 0.0, 1.0), C=glorot(256, 128, 7), K=256, N=128, name=CONFIG_NAMES[3])
    if idx == 4:
        s = 21 if scale >= 1.0 else max(10, 21 + int(np.floor(np.log2(scale))))
        A = rmat(s, (1 << s) * 8, seed=8)
        n = A.shape[0]
        return dict(op="gemm_spmm", A=A, B=uniform((n, 128), 9), C=uniform((128, 128), 10), K=128, N=128, name=CONFIG_NAMES[4])
    if idx == 5:
        g = 128 if scale >= 1.0 else max(8, int(round(128 * scale ** (1.0 / 3.0))))
        A = laplacian_3d(g)
        M = A.shape[0]
        return dict(op="spmm_spmm", A=A, B=A, C=uniform((M, 64), 11), K=0, N=64, name=CONFIG_NAMES[5])
    if idx == 6:
        M = max(256, int(262144 * scale))
        A = banded_random(M, 32, 16, seed=3)
        return dict(op="gemm_spmm", A=A, B=uniform((M, 128), 12), C=uniform((128, 128), 13), K=128, N=128, name=CONFIG_NAMES[6])
    if idx == 7:
        g = 128 if scale >= 1.0 else max(8, int(round(128 * scale ** (1.0 / 3.0))))
        A = box_stencil_3d(g)
        M = A.shape[0]
        return dict(op="spmm_spmm", A=A, B=A, C=uniform((M, 64), 14), K=0, N=64, name=CONFIG_NAMES[7])
    raise ValueError(f"unknown config {idx}")


def flops(cfg):
    """Algorithmic flops: GeMM-SpMM 2*M*K*N + 2*nnz*N; SpMM-SpMM 2*nnz(B)*N + 2*nnz(A)*N."""
    A, N = cfg["A"], cfg["N"]
    if cfg["op"] == "gemm_spmm":
        return 2.0 * A.shape[1] * cfg["K"] * N + 2.0 * A.nnz * N
    return 2.0 * cfg["B"].nnz * N + 2.0 * A.nnz * N


def algorithmic_bytes(cfg):
    """Compulsory HBM bytes of the fused product (the intermediate never leaves the chip,
    a sparse matrix used twice is read once): indices+values, row pointers, dense inputs,
    dense output."""
    A, N = cfg["A"], cfg["N"]
    M = A.shape[1]
    L = A.shape[0]
    if cfg["op"] == "gemm_spmm":
        K = cfg["K"]
        return 8.0 * A.nnz + 4.0 * (L + 1) + 4.0 * (M * K + K * N + L * N)
    B = cfg["B"]
    sparse = 8.0 * A.nnz + 4.0 * (L + 1)
    if B is not A:
        sparse += 8.0 * B.nnz + 4.0 * (B.shape[0] + 1)
    return sparse + 4.0 * (B.shape[1] * N + L * N)
