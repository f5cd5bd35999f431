"""Marching runs (fused SpMM-SpMM on 3D stencils) on the GPU, through the C ABI: the same bits as
the oracle -- every row is summed in CSR order out of LDS -- on cubes, on grids with unequal
sides, with random values, two strips of columns, accumulation and B != A in value."""
import numpy as np
import pytest
import scipy.sparse as sp

from test_gpu_parity import oracle_spmm_spmm, say

pytestmark = pytest.mark.gpu


def stencil_3d(nx, ny, nz, seed=None):
    """7-point stencil on an nx x ny x nz grid, x fastest; random values when a seed is given."""
    def t(n):
        e = np.ones(n)
        return sp.diags([-e[:-1], 2 * e, -e[:-1]], [-1, 0, 1])
    ix, iy, iz = sp.identity(nx), sp.identity(ny), sp.identity(nz)
    A = sp.csr_matrix(sp.kron(sp.kron(iz, iy), t(nx)) + sp.kron(sp.kron(iz, t(ny)), ix) + sp.kron(sp.kron(t(nz), iy), ix))
    A.eliminate_zeros()
    A.sort_indices()
    A = sp.csr_matrix((A.data.astype(np.float32), A.indices.astype(np.int32), A.indptr.astype(np.int32)), shape=A.shape)
    if seed is not None:
        A.data = np.random.default_rng(seed).uniform(-1, 1, A.nnz).astype(np.float32)
    return A


def march(tf, A, B, Cd, accumulate=False, D0=None, **kw):
    Ah = tf.CsrMatrix.from_scipy(A)
    Bh = Ah if B is A else tf.CsrMatrix.from_scipy(B)
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=Cd.shape[1], inner=Ah, march=1, **kw)
    S.validate()
    info = S.info()
    assert info["marched"] == 1 and info["n_fused_rows"] == A.shape[0] and info["n_writeback_rows"] == 0
    D = tf.DenseMatrix(A.shape[0], Cd.shape[1], D0) if D0 is not None else tf.DenseMatrix(A.shape[0], Cd.shape[1])
    if D0 is None:
        D.fill(float("nan"))
    tf.spmm_spmm(Ah, Bh, tf.DenseMatrix.from_numpy(Cd), D, S, accumulate=accumulate)
    tf.device_synchronize()
    return D.to_numpy(), info


@pytest.mark.parametrize("dims,N", [((12, 12, 12), 64), ((20, 20, 20), 64), ((40, 40, 40), 64), ((9, 14, 31), 64),
                                    ((33, 5, 17), 64), ((16, 16, 40), 128), ((11, 23, 8), 192)])
def test_march_bit_exact(gpu, tf, orc, dims, N):
    say(f"march {dims} N={N}")
    nx, ny, nz = dims
    A = stencil_3d(nx, ny, nz, seed=7)
    Cd = tf.workloads.uniform((A.shape[0], N), 8)
    want = oracle_spmm_spmm(orc, A, A, Cd)
    got, info = march(tf, A, A, Cd)              # the grid is found from the pattern
    assert np.array_equal(got, want), (dims, N, info)
    got, info = march(tf, A, A, Cd, compute_units=16)   # fewer, longer runs
    assert np.array_equal(got, want), (dims, N, info)


@pytest.mark.parametrize("dims,N", [((300, 1, 90), 64), ((128, 1, 128), 128), ((10, 9, 700), 64)])
def test_march_flat_and_tall_grids(gpu, tf, orc, dims, N):
    """A 5-point stencil on a 2D grid (found from its two distances; the runs walk the grid's lines, 64 points of
    a line at a time) and a grid with more planes than a run's table of iterations holds (cut into several runs
    along z): the same bits as the oracle."""
    say(f"march {dims} N={N}")
    nx, ny, nz = dims
    A = stencil_3d(nx, ny, nz, seed=17)
    Cd = tf.workloads.uniform((A.shape[0], N), 18)
    want = oracle_spmm_spmm(orc, A, A, Cd)
    got, info = march(tf, A, A, Cd)
    assert np.array_equal(got, want), (dims, N, info)
    if ny == 1:
        assert info["march_tile_y"] == 1 and info["march_tile_x"] > 8, info
    if nz > 254:
        got, info = march(tf, A, A, Cd, compute_units=4)   # few compute units: the cut comes from the table's size
        assert np.array_equal(got, want), (dims, N, info)
        assert info["n_tiles"] > 4, info


def test_march_tiles_hints_and_operands(gpu, tf, orc):
    say("march: tile sizes, grid hints, B != A, accumulate")
    nx, ny, nz = 24, 18, 30
    A = stencil_3d(nx, ny, nz, seed=9)
    M, N = A.shape[0], 64
    Cd = tf.workloads.uniform((M, N), 10)
    want = oracle_spmm_spmm(orc, A, A, Cd)
    for tile in ((8, 8), (4, 4), (8, 3), (5, 7), (3, 2)):
        got, info = march(tf, A, A, Cd, march_tile=tile)
        assert (info["march_tile_x"], info["march_tile_y"]) == tile
        assert np.array_equal(got, want), tile
    # a wrong grid (same number of points) only changes how rows are dealt to runs: the schedule is
    # either refused or still exact
    for grid in ((nx, ny, nz), (ny, nx, nz), (nx * ny, 1, nz), (12, 36, 30)):
        try:
            got, info = march(tf, A, A, Cd, grid=grid)
        except tf.TileFusionError as e:
            assert e.status == -5
            continue
        assert np.array_equal(got, want), grid
    B = A.copy()
    B.data = tf.workloads.uniform((A.nnz,), 11)
    got, _ = march(tf, A, B, Cd)
    assert np.array_equal(got, oracle_spmm_spmm(orc, A, B, Cd))
    D0 = tf.workloads.uniform((M, N), 12)
    got, _ = march(tf, A, A, Cd, accumulate=True, D0=D0)
    assert orc.rel_err(got, D0.astype(np.float64) + want) <= 1e-6
    # the library's own Laplacian (the benchmark's matrix, scaled down), default options: marching is chosen
    L = tf.workloads.laplacian_3d(30)
    Lh = tf.CsrMatrix.from_scipy(L)
    S = tf.inspector(Lh, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Lh)
    assert S.info()["marched"] == 1
    S = tf.inspector(Lh, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Lh, march=-1)
    assert S.info()["marched"] == 0 and S.info()["n_fused_rows"] == 0


def test_march_full_size_all_ones_exact(gpu, tf):
    """The benchmark's 128^3 Laplacian with an all-ones dense operand (the reference's own input,
    fusion/example/SpMM_SpMM_Demo_Utils.h:53-59): integers throughout, so D must equal the 7-point
    stencil applied twice on the grid, exactly, at full size; and with the benchmark's uniform C,
    against float64 on a sample of rows."""
    say("march 128^3 all ones")
    g, N = 128, 64
    A = tf.workloads.laplacian_3d(g)
    got, info = march(tf, A, A, np.ones((g ** 3, N), np.float32))
    assert (info["march_tile_x"], info["march_tile_y"]) == (8, 8) and info["n_tiles"] == 256

    def st(u):
        out = 6.0 * u
        out[:, :, 1:] -= u[:, :, :-1]; out[:, :, :-1] -= u[:, :, 1:]
        out[:, 1:, :] -= u[:, :-1, :]; out[:, :-1, :] -= u[:, 1:, :]
        out[1:, :, :] -= u[:-1, :, :]; out[:-1, :, :] -= u[1:, :, :]
        return out
    want = st(st(np.ones((g, g, g), np.float32))).reshape(-1)
    assert np.array_equal(got, np.repeat(want[:, None], N, axis=1))
    Cd = tf.workloads.uniform((g ** 3, N), 11)
    got, _ = march(tf, A, A, Cd)
    rows = np.random.default_rng(13).choice(g ** 3, 20000, replace=False)
    T = A.astype(np.float64) @ Cd.astype(np.float64)
    ref = A[rows].astype(np.float64) @ T
    assert np.abs(got[rows] - ref).max() / np.abs(ref).max() <= 1e-5


def box_stencil(nx, ny, nz, corners, seed):
    """The stencil of all neighbours within one step in every direction on an nx x ny x nz grid, x fastest:
    27 points -- or 19 without the eight corners of the cube.  Random values."""
    def t(n):
        e = np.ones(n)
        return sp.diags([e[:-1], e, e[:-1]], [-1, 0, 1])

    def off(n):
        e = np.ones(n)
        return sp.diags([e[:-1], e[:-1]], [-1, 1])
    A = sp.csr_matrix(sp.kron(sp.kron(t(nz), t(ny)), t(nx)))
    if not corners:
        A = A - sp.csr_matrix(sp.kron(sp.kron(off(nz), off(ny)), off(nx)))
        A.eliminate_zeros()
    A.sort_indices()
    A = sp.csr_matrix((A.data.astype(np.float32), A.indices.astype(np.int32), A.indptr.astype(np.int32)), shape=A.shape)
    A.data = np.random.default_rng(seed).uniform(-1, 1, A.nnz).astype(np.float32)
    return A


@pytest.mark.parametrize("dims,corners,N", [((12, 12, 12), True, 64), ((20, 17, 9), True, 64), ((9, 14, 31), False, 64),
                                            ((24, 24, 24), True, 128), ((40, 40, 40), True, 64), ((17, 6, 23), False, 192)])
def test_march_wide_stencils_bit_exact(gpu, tf, orc, dims, corners, N):
    """27- and 19-point stencils: rows of more than eight entries march with ELL rows of 32 pairs, a lane of the
    16-lane group holding two, passed on by DPP row broadcasts.  The same bits as the oracle, the grid found from
    the pattern's distances."""
    say(f"march wide {dims} corners={corners} N={N}")
    A = box_stencil(*dims, corners, seed=21)
    assert np.diff(A.indptr).max() == (27 if corners else 19)
    Cd = tf.workloads.uniform((A.shape[0], N), 22)
    want = oracle_spmm_spmm(orc, A, A, Cd)
    got, info = march(tf, A, A, Cd)
    assert np.array_equal(got, want), (dims, N, info)
    got, info = march(tf, A, A, Cd, compute_units=16)
    assert np.array_equal(got, want), (dims, N, info)


def test_march_wide_accumulate_other_values_and_flat_grid(gpu, tf, orc):
    """Wide rows with D accumulated into, with an inner matrix of the same pattern and other values, and a 9-point
    stencil on a flat grid (rows of nine entries: the narrowest of the wide kernels)."""
    say("march wide: accumulate, B != A, 9 points on a flat grid")
    A = box_stencil(14, 11, 10, True, seed=23)
    B = A.copy()
    B.data = np.random.default_rng(24).uniform(-1, 1, B.nnz).astype(np.float32)
    M = A.shape[0]
    Cd = tf.workloads.uniform((M, 64), 25)
    D0 = tf.workloads.uniform((M, 64), 26)
    want = oracle_spmm_spmm(orc, A, B, Cd)
    got, _ = march(tf, A, B, Cd)
    assert np.array_equal(got, want)
    got, _ = march(tf, A, B, Cd, accumulate=True, D0=D0)
    assert orc.rel_err(got, want.astype(np.float64) + D0) <= 1e-6
    F = box_stencil(200, 1, 60, True, seed=27)     # nz x nx grid of 9-point rows
    assert np.diff(F.indptr).max() == 9
    Cf = tf.workloads.uniform((F.shape[0], 64), 28)
    got, info = march(tf, F, F, Cf)
    assert np.array_equal(got, oracle_spmm_spmm(orc, F, F, Cf)), info

