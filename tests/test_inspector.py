"""The gfx950 inspector (tf_inspect) on the CPU: schedules are checked exactly by an
independent validator written here, by the library's own validator, and against
hand-derived fused sets on banded and stencil patterns."""
import numpy as np
import pytest
import scipy.sparse as sp


def validate(view, info, A, lds_budget):
    """Independent of the library: every first-op row owned once, every second-op row
    scheduled once, fused rows read only rows their tile computes, remainder rows read
    only rows some tile writes back, slabs fit the LDS budget."""
    L, M = A.shape
    tr, wb = view["tile_range"], view["writeback"]
    nt = len(tr)
    assert view["n1_"] == 2 and view["ptr1_"][0] == 0 and view["ptr1_"][1] == nt
    P = view["ptr1_"][2]
    ptr2, kb, ids, typ = view["ptr2_"], view["ker_begin_"], view["id_"], view["type_"]
    assert len(ptr2) == P + 1 and ptr2[0] == 0 and ptr2[P] == len(ids) == M + L
    assert np.array_equal(np.sort(ids[typ == 0]), np.arange(M))
    assert np.array_equal(np.sort(ids[typ == 1]), np.arange(L))
    stored = np.zeros(M, bool)
    fused_rows = 0
    end = 0
    for t in range(nt):
        pb, pe, ob, oe = tr[t]
        assert ob == end and oe > ob and pb <= ob and pe >= oe and 0 <= pb and pe <= M
        end = oe
        own = ids[ptr2[t]:kb[2 * t]]
        fused = ids[kb[2 * t]:kb[2 * t + 1]]
        assert kb[2 * t + 1] == ptr2[t + 1]
        assert np.array_equal(own, np.arange(ob, oe))
        assert np.all(typ[ptr2[t]:kb[2 * t]] == 0) and np.all(typ[kb[2 * t]:kb[2 * t + 1]] == 1)
        if len(fused) and info["streamed"]:
            # a streamed run is produced 64 rows a step into a ring of ring_rows rows: a row of
            # step q is computed while rows pb + 64q .. are produced, so all its columns come from
            # earlier steps and lie within the last ring_rows - 64 rows
            ring = info["ring_rows"]
            assert ring >= 256 and ring % 64 == 0 and ring * (info["N"] + 4) * 4 <= lds_budget
            st = view["tile_step"][t]
            steps = -(-(pe - pb) // 64)
            sp_ = view["step_ptr"][st:st + steps + 2]
            assert st >= 0 and sp_[0] == 0 and sp_[-1] == len(fused) and np.all(np.diff(sp_) >= 0)
            for q in range(steps + 1):
                for i in fused[sp_[q]:sp_[q + 1]]:
                    cols = A.indices[A.indptr[i]:A.indptr[i + 1]]
                    assert 0 < len(cols) <= 32
                    qc = (cols - pb) // 64
                    assert qc.max() <= q - 1 and qc.min() >= q - ring // 64 + 1, f"row {i} step {q}"
        elif len(fused):
            assert (pe - pb) * info["N"] * 4 <= lds_budget
        for i in fused:
            cols = A.indices[A.indptr[i]:A.indptr[i + 1]]
            if len(cols):
                assert cols.min() >= pb and cols.max() < pe, f"fused row {i} leaves tile {t}"
        fused_rows += len(fused)
        assert ob <= wb[t][0] <= wb[t][1] <= oe
        stored[wb[t][0]:wb[t][1]] = True
    assert end == M
    assert fused_rows == info["n_fused_rows"] and fused_rows + info["n_remainder_rows"] == L
    for p in range(nt, P):
        rows = ids[ptr2[p]:ptr2[p + 1]]
        assert 0 < len(rows) <= 64 and kb[2 * p] == ptr2[p] and kb[2 * p + 1] == ptr2[p + 1]
        for i in rows:
            cols = A.indices[A.indptr[i]:A.indptr[i + 1]]
            assert np.all(stored[cols]), f"remainder row {i} reads a row nobody stores"
    # rows actually stored: at least every row a remainder row reads, at most the write-back ranges
    needed = np.zeros(M, bool)
    for p in range(nt, P):
        for i in ids[ptr2[p]:ptr2[p + 1]]:
            needed[A.indices[A.indptr[i]:A.indptr[i + 1]]] = True
    assert int(needed.sum()) <= info["n_writeback_rows"] <= int(sum(b - a for a, b in wb))


def inspect(tf, A, **kw):
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, 1, **kw)
    S.validate()
    return S, S.view(), S.info()


@pytest.mark.parametrize("idx,scale", [(1, 1.0), (2, 0.1), (3, 0.02), (4, 2.0 ** -7), (5, 0.004)])
def test_configs_validate(tf, idx, scale):
    cfg = tf.workloads.make_config(idx, scale)
    op = tf.OP_GEMM_SPMM if cfg["op"] == "gemm_spmm" else tf.OP_SPMM_SPMM
    for budget in (32768, 65536, 163840):
        S, view, info = inspect(tf, cfg["A"], op=op, N=cfg["N"], K=cfg["K"], lds_budget_bytes=budget)
        validate(view, info, cfg["A"], budget)


def test_banded_halo_fuses_everything(tf):
    """Half-bandwidth 16: with recomputation every row fuses and nothing is written back;
    each tile computes its owned rows plus at most 16 halo rows per side."""
    A = tf.workloads.banded_random(4096, 32, 16, seed=3)
    S, view, info = inspect(tf, A, op=tf.OP_SPMM_SPMM, N=128, lds_budget_bytes=65536)
    validate(view, info, A, 65536)
    assert info["n_fused_rows"] == 4096 and info["n_remainder_rows"] == 0 and info["n_writeback_rows"] == 0
    tr = view["tile_range"]
    assert np.all(tr[:, 2] - tr[:, 0] <= 16) and np.all(tr[:, 1] - tr[:, 3] <= 16)
    assert np.all(tr[:, 1] - tr[:, 0] <= 65536 // (128 * 4))


def test_no_recomputation_matches_reference_rule(tf):
    """max_redundancy = 1 is the reference's tiling: a row fuses iff all its columns are
    rows of its own tile (Fusion_Inspector.h:885-891, without the sorted-columns shortcut)."""
    n = 32
    A = tf.workloads.laplacian_2d(n)
    S, view, info = inspect(tf, A, op=tf.OP_SPMM_SPMM, N=64, lds_budget_bytes=65536, tile_rows=256, max_redundancy=1.0)
    validate(view, info, A, 65536)
    tr = view["tile_range"]
    assert np.array_equal(tr[:, 0], tr[:, 2]) and np.array_equal(tr[:, 1], tr[:, 3])
    assert np.all(tr[:, 3] - tr[:, 2] == 256)
    ids, kb = view["id_"], view["ker_begin_"]
    M = n * n
    for t, (s, e, _, _) in enumerate(tr):
        want = [i for i in range(s, e) if (i - n < 0 or i - n >= s) and (i + n >= M or i + n < e)
                and (i % n == 0 or i - 1 >= s) and (i % n == n - 1 or i + 1 < e)]
        assert ids[kb[2 * t]:kb[2 * t + 1]].tolist() == want
    # remainder rows = n rows either side of every interior boundary -> their reads force write-back
    assert info["n_remainder_rows"] == 2 * n * (len(tr) - 1)
    assert info["n_writeback_rows"] > 0


def test_unsorted_columns_and_empty_rows(tf):
    """Columns in any order, rows without entries, and a row that reaches across the
    matrix (never fusable) are all scheduled exactly once."""
    rng = np.random.default_rng(0)
    M = 700
    rows, cols = [], []
    for i in range(M):
        if i % 7 == 3:
            continue
        c = np.unique(np.clip(i + rng.integers(-5, 6, 4), 0, M - 1))
        rng.shuffle(c)
        rows += [i] * len(c)
        cols += c.tolist()
    rows += [350, 350]
    cols += [0, M - 1]
    A = sp.csr_matrix((np.ones(len(rows), np.float32), (rows, cols)), shape=(M, M))
    A.has_sorted_indices = False
    perm_A = A.copy()
    for i in range(M):  # scramble each row's column order
        s, e = perm_A.indptr[i], perm_A.indptr[i + 1]
        p = rng.permutation(e - s)
        perm_A.indices[s:e] = perm_A.indices[s:e][p]
    S, view, info = inspect(tf, perm_A, op=tf.OP_SPMM_SPMM, N=32, lds_budget_bytes=16384)
    validate(view, info, perm_A, 16384)
    assert 350 in view["id_"][view["ptr2_"][view["ptr1_"][1]]:]  # the far-reaching row is a remainder row
    assert info["n_remainder_rows"] >= 1


def test_long_rows_are_chunked(tf):
    M = 4096
    hub = sp.csr_matrix((np.ones(3000, np.float32), (np.zeros(3000, int), np.arange(3000))), shape=(M, M))
    A = sp.csr_matrix(hub + sp.identity(M, dtype=np.float32, format="csr"))
    S, view, info = inspect(tf, A, op=tf.OP_SPMM_SPMM, N=64, long_row_nnz=512)
    validate(view, info, A, 65536)
    assert info["n_long_rows"] == 1 and info["n_long_chunks"] == 3  # ceil(3000 / max(512, 1024))


def test_rectangular_and_bad_arguments(tf):
    A = sp.random(300, 200, density=0.02, format="csr", random_state=np.random.default_rng(1), dtype=np.float32)
    S, view, info = inspect(tf, A, op=tf.OP_SPMM_SPMM, N=16)
    validate(view, info, A, 65536)
    A2 = sp.random(200, 300, density=0.02, format="csr", random_state=np.random.default_rng(2), dtype=np.float32)
    S, view, info = inspect(tf, A2, op=tf.OP_SPMM_SPMM, N=16)
    validate(view, info, A2, 65536)
    Ah = tf.CsrMatrix.from_scipy(A)
    for kw in (dict(op=7, N=16), dict(op=tf.OP_SPMM_SPMM, N=0), dict(op=tf.OP_GEMM_SPMM, N=64, K=0),
               dict(op=tf.OP_SPMM_SPMM, N=16, lds_budget_bytes=1 << 20), dict(op=tf.OP_SPMM_SPMM, N=4096, lds_budget_bytes=16384)):
        with pytest.raises(tf.TileFusionError) as e:
            tf.inspector(Ah, 1, **kw)
        assert e.value.status == -1
    # GeMM-SpMM of any width: the schedule is built for column panels of a width the MFMA kernels take
    # (48 -> one panel of 64, 300 -> two of 160, 700 -> three of 256) and says so in its workspace
    sq = tf.CsrMatrix.from_scipy(A2[:, :200])
    for N, panel in ((48, 64), (300, 160), (700, 256), (7, 32)):
        Sp = tf.inspector(sq, 1, op=tf.OP_GEMM_SPMM, N=N, K=64)
        Sp.validate()
        assert Sp.info()["N"] == N and Sp.info()["workspace_bytes"] >= (200 + 64) * panel * 4
    Sq = tf.inspector(tf.CsrMatrix.from_scipy(A2[:, :200]), 1, op=tf.OP_GEMM_SPMM, N=64, K=20)  # any K: padded to 24
    assert Sq.info()["K"] == 20 and Sq.info()["workspace_bytes"] >= (200 + 64) * 24 * 4
    bad = tf.CsrMatrix(4, 4, [0, 1, 2, 3, 4], [0, 1, 9, 3], [1, 1, 1, 1])
    with pytest.raises(tf.TileFusionError):
        tf.inspector(bad, 1, op=tf.OP_SPMM_SPMM, N=8)


def test_validator_rejects_a_schedule_for_another_pattern(tf):
    A = tf.workloads.banded_random(1024, 32, 16, seed=1)
    B = tf.workloads.laplacian_2d(32)
    S = tf.inspector(tf.CsrMatrix.from_scipy(A), 1, op=tf.OP_SPMM_SPMM, N=64)
    with pytest.raises(tf.TileFusionError) as e:
        S.validate(tf.CsrMatrix.from_scipy(B))
    assert e.value.status == -4
    A2 = A.copy()
    A2.indices[A2.indptr[500]] = 0  # same size, one dependence moved far away
    with pytest.raises(tf.TileFusionError) as e:
        S.validate(tf.CsrMatrix.from_scipy(A2))
    assert e.value.status == -4 and "row 500" in str(e.value)


def test_windowed_tiles(tf):
    """With the inner pattern given, banded and narrow-grid patterns get windowed tiles:
    every row fused, nothing written back, and the window of C recorded per tile covers
    every column the tile's producer rows read."""
    for A, N in ((tf.workloads.banded_random(4096, 32, 16, seed=3), 128), (tf.workloads.laplacian_2d(48), 64)):
        Ah = tf.CsrMatrix.from_scipy(A)
        S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=N, inner=Ah, wide_strips=-1)  # the lane-group kernel's tiles
        S.validate()
        info, view = S.info(), S.view()
        assert info["windowed"] == 1 and info["strip_cols"] == 32
        assert info["n_fused_rows"] == A.shape[0] and info["n_writeback_rows"] == 0
        assert info["lds_bytes"] <= 81920
        validate(view, info, A, 163840)
    # a pattern whose rows reach across the matrix cannot be windowed
    R = tf.workloads.erdos_renyi_gcn(4000, 10.0, seed=5)
    Rh = tf.CsrMatrix.from_scipy(R)
    assert tf.inspector(Rh, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Rh).info()["windowed"] == 0


def test_wide_strip_tiles(tf):
    """With the inner pattern given and N a multiple of 64, windowed tiles are built for the
    64-column kernel, one per compute unit (at least 64 rows): LDS holds row pointers, window
    and slab (no entries), up to 160 KB; any explicit strip, tile or LDS choice keeps the
    lane-group kernel's tiles."""
    A = tf.workloads.banded_random(4096, 32, 16, seed=3)
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=128, inner=Ah, compute_units=16)
    S.validate()
    info, view = S.info(), S.view()
    assert info["windowed"] == 1 and info["wide_strips"] == 1 and info["strip_cols"] == 64 and info["n_tiles"] == 16
    assert info["n_fused_rows"] == 4096 and info["n_writeback_rows"] == 0
    tr = view["tile_range"].reshape(-1, 4)
    P = int((tr[:, 1] - tr[:, 0]).max())  # producer rows of the largest tile: window and slab each hold at least as many
    assert 4 * 64 * 2 * P <= info["lds_bytes"] <= 163840
    validate(view, info, A, 163840)
    assert tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=128, inner=Ah, compute_units=256).info()["n_tiles"] == 64  # 64 rows each
    for kw in (dict(compute_units=16, strip_cols=32), dict(compute_units=16, tile_rows=128),
               dict(compute_units=16, lds_budget_bytes=65536), dict(compute_units=16, wide_strips=-1)):
        assert tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=128, inner=Ah, **kw).info()["wide_strips"] == 0, kw
    assert tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=96, inner=Ah, compute_units=16).info()["wide_strips"] == 0
    assert tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Ah, compute_units=64, wide_strips=1).info()["wide_strips"] == 1
    # where LDS allows fewer rows than one compute unit's share, the tiles are sized for a whole number of turns
    for cu in (2, 3, 4, 6, 7):
        Sm = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=128, inner=Ah, compute_units=cu)
        Sm.validate()
        n = Sm.info()["n_tiles"]
        assert n > cu and n % cu == 0 and Sm.info()["n_fused_rows"] == 4096, (cu, n)


def test_long_rows_by_column_partition(tf):
    """long_row_partition: the long rows' entries regrouped by the XCD partition of their column
    (the most-read intermediate rows, an L2's worth per XCD) into segments of at most 64;
    every entry once, CSR order inside a segment, a column read through one partition only --
    checked by the library's validator and recounted here from the info."""
    cfg = tf.workloads.make_config(4, 2.0 ** -5)
    A = cfg["A"]
    Ah = tf.CsrMatrix.from_scipy(A)
    base = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128)
    assert base.info()["long_row_hot_cols"] == 0 and base.info()["n_long_rows"] > 0
    S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128, long_row_partition=1)
    S.validate()
    info = S.info()
    rl = np.diff(A.indptr)
    # (left to the library, the threshold is 32 entries for rows in chunks and 64 for rows regrouped by partition)
    assert base.info()["n_long_rows"] == int((rl > 32).sum()) and info["n_long_rows"] == int((rl > 64).sum())
    S32 = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128, long_row_partition=1, long_row_nnz=32)
    S32.validate()
    assert S32.info()["n_long_rows"] == base.info()["n_long_rows"]
    long_nnz = int(rl[rl > 64].sum())
    assert 0 < info["long_row_hot_cols"] <= 8 * (12 << 20) // (128 * 4)
    # at least one segment per 64 entries, and the eight hot lists are padded to whole workgroups
    assert info["n_long_chunks"] >= long_nnz // 64 and info["n_long_chunks"] % 1 == 0
    assert info["workspace_bytes"] >= info["n_long_chunks"] * 128 * 4 + long_nnz * 4
    assert tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128, long_row_partition=-1).info()["long_row_hot_cols"] == 0
    # SpMM-SpMM takes the same remainder path
    S2 = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64, long_row_partition=1)
    S2.validate()
    assert S2.info()["long_row_hot_cols"] > 0


def test_xcd_chunk_is_the_callers_choice(tf):
    A = tf.workloads.laplacian_3d(40)
    Ah = tf.CsrMatrix.from_scipy(A)
    assert tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64).info()["xcd_chunk_rows"] == 0
    assert tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64, xcd_chunk_rows=512).info()["xcd_chunk_rows"] == 512
    assert tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64, xcd_chunk_rows=-1).info()["xcd_chunk_rows"] == -1


def test_streamed_runs(tf):
    """GeMM-SpMM on a long banded matrix: one run per compute unit, every row fused, rows listed
    step by step at no more than 64 a step, no halo beyond the band; denser and far-reaching
    rows are left to the remainder and their intermediate rows written back."""
    M = 40000
    A = tf.workloads.banded_random(M, 32, 16, seed=5)
    S, view, info = inspect(tf, A, op=tf.OP_GEMM_SPMM, N=128, K=128, compute_units=256)
    validate(view, info, A, 163840)
    assert info["streamed"] == 1 and info["ring_rows"] == 256
    assert info["n_fused_rows"] == M and info["n_writeback_rows"] == 0
    tr = view["tile_range"]
    assert len(tr) == 256 and np.all(tr[:, 2] - tr[:, 0] <= 16) and np.all(tr[:, 1] - tr[:, 3] <= 16)  # a run per compute unit
    assert set((tr[:, 3] - tr[:, 2]).tolist()) <= {156, 157}
    for t in range(len(tr)):
        st = view["tile_step"][t]
        steps = -(-(tr[t][1] - tr[t][0]) // 64)
        assert np.all(np.diff(view["step_ptr"][st:st + steps + 1]) <= 64)
    # a matrix too short to give every compute unit a run keeps the tile kernel
    S2, _, info2 = inspect(tf, tf.workloads.banded_random(4096, 32, 16, seed=5), op=tf.OP_GEMM_SPMM, N=128, K=128, compute_units=256)
    assert info2["streamed"] == 0 and info2["n_fused_rows"] == 4096
    # rows the stream cannot take: more than 32 entries, or a column far away
    rng = np.random.default_rng(6)
    B = A.tolil()
    dense_rows = rng.choice(M, 50, replace=False)
    for i in dense_rows:
        lo = max(0, i - 30)
        B[i, lo:lo + 40] = 1.0
    far_rows = rng.choice(M, 50, replace=False)
    for i in far_rows:
        B[i, (i + M // 2) % M] = 2.0
    B = sp.csr_matrix(B, dtype=np.float32)
    S3, view3, info3 = inspect(tf, B, op=tf.OP_GEMM_SPMM, N=128, K=128, compute_units=256)
    validate(view3, info3, B, 163840)
    out = set(dense_rows.tolist()) | set(far_rows.tolist())
    assert info3["streamed"] == 1 and info3["n_remainder_rows"] == len(out) and info3["n_writeback_rows"] > 0
    # wider rows and narrower rings: N = 32 holds a ring of 1024 rows, and K = 256 halves the consumers
    for N, K in ((32, 64), (64, 256), (96, 8)):
        S4, view4, info4 = inspect(tf, A, op=tf.OP_GEMM_SPMM, N=N, K=K, compute_units=256)
        validate(view4, info4, A, 163840)
        assert info4["streamed"] == 1 and info4["n_fused_rows"] == M


# ---- options struct, pattern fingerprint, inner-pattern check --------------------------------

def test_opts_struct_size_is_honoured(tf):
    """A caller compiled against an older, shorter tf_inspect_opts passes its own size: the
    library reads only that many bytes and takes defaults for the rest; 0 is rejected."""
    import ctypes as C
    from importlib import import_module
    b = import_module("tile-fusion_amd.binding")
    A = tf.workloads.banded_random(2000, 32, 16, seed=3)
    Ah = tf.CsrMatrix.from_scipy(A)
    full = b.InspectOpts(C.sizeof(b.InspectOpts), tf.OP_SPMM_SPMM, 64)
    h = C.c_void_p()
    assert b.lib().tf_inspect(A.shape[0], A.shape[1], Ah._pp, Ah._pi, C.byref(full), C.byref(h)) == 0
    ref = b.FusedSchedule(h, Ah).info()
    # the same options in a buffer that ends right after K, followed by garbage the library must not read
    short_size = b.InspectOpts.K.offset + C.sizeof(C.c_int)
    raw = (C.c_ubyte * C.sizeof(b.InspectOpts))(*([0xAB] * C.sizeof(b.InspectOpts)))
    C.memmove(raw, C.byref(full), short_size)
    C.cast(raw, C.POINTER(C.c_size_t))[0] = short_size
    h2 = C.c_void_p()
    assert b.lib().tf_inspect(A.shape[0], A.shape[1], Ah._pp, Ah._pi, C.cast(raw, C.POINTER(b.InspectOpts)), C.byref(h2)) == 0
    assert b.FusedSchedule(h2, Ah).info() == ref
    zero = b.InspectOpts(0, tf.OP_SPMM_SPMM, 64)
    h3 = C.c_void_p()
    assert b.lib().tf_inspect(A.shape[0], A.shape[1], Ah._pp, Ah._pi, C.byref(zero), C.byref(h3)) == -1
    assert b"struct_size" in b.lib().tf_last_error_string()


def test_out_struct_size_is_honoured(tf):
    """The structs the library fills in carry the caller's size too: a caller compiled against a
    struct one field shorter gets exactly its bytes, a canary right behind them stays intact, and
    a size below the struct's first version (a forgotten 0) is refused."""
    import ctypes as C
    from importlib import import_module
    b = import_module("tile-fusion_amd.binding")
    A = tf.workloads.banded_random(2000, 32, 16, seed=3)
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, op=tf.OP_GEMM_SPMM, N=128, K=128)
    lib = b.lib()

    def call_short(struct, fn, handle, cut_field):
        """Calls fn(handle, buf) with buf = the struct cut right after `cut_field`, 0xAB behind it."""
        full = struct(C.sizeof(struct))
        assert fn(handle, C.byref(full)) == 0
        fld = getattr(struct, cut_field)
        short = fld.offset + fld.size
        assert short < C.sizeof(struct)
        raw = (C.c_ubyte * (C.sizeof(struct) + 64))(*([0xAB] * (C.sizeof(struct) + 64)))
        C.cast(raw, C.POINTER(C.c_size_t))[0] = short
        assert fn(handle, C.cast(raw, C.POINTER(struct))) == 0, lib.tf_last_error_string()
        assert bytes(raw[C.sizeof(C.c_size_t):short]) == bytes(full)[C.sizeof(C.c_size_t):short]
        assert all(x == 0xAB for x in raw[short:]), "the library wrote behind the caller's struct"
        assert C.cast(raw, C.POINTER(C.c_size_t))[0] == short
        zero = struct(0)
        assert fn(handle, C.byref(zero)) == -1 and b"struct_size" in lib.tf_last_error_string()

    # the last fields of today's structs are cut off as a later header's would be
    last_info = b.ScheduleInfo._fields_[-1][0]
    prev_info = b.ScheduleInfo._fields_[-2][0]
    # (a struct cut before the end of its first version is refused, so cut only what came later)
    first_version_end = "march_slots"
    if last_info != first_version_end:
        call_short(b.ScheduleInfo, lib.tf_schedule_get_info, S.h, prev_info if prev_info != first_version_end else first_version_end)
    too_short = b.ScheduleInfo(b.ScheduleInfo.march_slots.offset)  # ends before march_slots
    assert lib.tf_schedule_get_info(S.h, C.byref(too_short)) == -1
    # a struct LONGER than the library's (a newer caller): only the library's bytes are written
    class Longer(C.Structure):
        _fields_ = b.ScheduleView._fields_ + [("future", C.c_longlong * 8)]   # (8-byte fields: behind the struct's tail padding)
    v = Longer(C.sizeof(Longer))
    for q in range(8):
        v.future[q] = 0x5A5A5A5A5A5A
    assert lib.tf_schedule_get_view(S.h, C.cast(C.byref(v), C.POINTER(b.ScheduleView))) == 0
    assert v.n1 == 2 and all(v.future[q] == 0x5A5A5A5A5A5A for q in range(8)) and v.struct_size == C.sizeof(Longer)
    for struct, fn in ((b.ScheduleView, lib.tf_schedule_get_view), (b.Profile, lib.tf_schedule_get_profile)):
        zero = struct(0)
        assert fn(S.h, C.byref(zero)) == -1 and b"struct_size" in lib.tf_last_error_string()


def test_pattern_hash(tf):
    A = tf.workloads.banded_random(1000, 32, 16, seed=3)
    h = tf.pattern_hash(A)
    assert h != 0 and h == tf.pattern_hash(A.copy()) == tf.pattern_hash(tf.CsrMatrix.from_scipy(A))
    B = A.copy()
    B.data[:] = 7.0                      # values do not enter
    assert tf.pattern_hash(B) == h
    B = A.copy()
    B.indices[5], B.indices[6] = B.indices[6], B.indices[5]   # same entries of the row, other order
    assert tf.pattern_hash(B) != h
    B = tf.workloads.banded_random(1000, 32, 16, seed=4)       # same shape and entry count
    assert B.nnz == A.nnz and tf.pattern_hash(B) != h
    assert tf.pattern_hash(A[:999]) != h


def test_validate_checks_windows_against_the_inner_pattern(tf):
    A = tf.workloads.banded_random(4000, 32, 16, seed=3)
    Ah = tf.CsrMatrix.from_scipy(A)
    for kw in (dict(), dict(wide_strips=-1, strip_cols=32)):
        S = tf.inspector(Ah, op=tf.OP_SPMM_SPMM, N=128, inner=Ah, **kw)
        assert S.info()["windowed"] == 1
        S.validate()                       # windows hold every row of C the producer rows read
        other = tf.CsrMatrix.from_scipy(tf.workloads.banded_random(4000, 32, 16, seed=9))
        S._inner = other                   # same shape and entry count, another pattern
        with pytest.raises(tf.TileFusionError) as e:
            S.validate()
        assert e.value.status == -4 and "inner pattern" in str(e.value)
        S._inner = None
        with pytest.raises(tf.TileFusionError) as e:
            S.validate()
        assert e.value.status == -1


# ---- marching runs: the validator must reject what does not match --------------------------------

def _moved_column(A, row, k, new_col):
    B = A.copy()
    B.indices = B.indices.copy()
    B.indices[B.indptr[row] + k] = new_col
    return B


def test_march_validator_rejects_other_patterns(tf):
    """A marching schedule replayed against a pattern it was not built from: one column of one row
    moved (in A, in the inner matrix, or in both), an entry moved from one row to another (one row
    longer, one shorter, same entry count), two columns of a row swapped -- each must be refused with
    TF_ESCHEDULE, and the pattern it was built from must pass before and after."""
    n = 12
    A = tf.workloads.laplacian_3d(n)
    M = A.shape[0]
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Ah, march=1)
    info = S.info()
    assert info["marched"] == 1 and info["march_declined"] == 0
    S.validate()
    mid = (n // 2 * n + n // 2) * n + n // 2           # an interior point: 7 entries, columns sorted
    assert A.indptr[mid + 1] - A.indptr[mid] == 7
    far = _moved_column(A, mid, 6, mid + n * n + 1)    # its +z neighbour replaced by that one's +x neighbour
    near = _moved_column(A, mid, 4, mid + 2)           # its +x neighbour replaced by the next point
    swapped = A.copy(); swapped.indices = swapped.indices.copy()
    s0 = swapped.indptr[mid]
    swapped.indices[s0 + 1], swapped.indices[s0 + 2] = swapped.indices[s0 + 2], swapped.indices[s0 + 1]
    # an entry moved from row `mid` to the corner row 0 (3 + 1 entries -> 5, 7 -> 6), same entry count
    lil = A.tolil(); lil[mid, mid + 1] = 0; lil[0, 5] = -1.0
    longer = sp.csr_matrix(lil); longer.eliminate_zeros(); longer.sort_indices()
    longer = sp.csr_matrix((longer.data.astype(np.float32), longer.indices.astype(np.int32), longer.indptr.astype(np.int32)), shape=A.shape)
    assert longer.nnz == A.nnz
    for name, other in (("far column", far), ("near column", near), ("swapped columns", swapped), ("longer row", longer)):
        Oh = tf.CsrMatrix.from_scipy(other)
        for outer, inner in ((Oh, Ah), (Ah, Oh), (Oh, Oh)):
            S._inner = inner
            with pytest.raises(tf.TileFusionError) as e:
                S.validate(outer)
            assert e.value.status == -4, (name, str(e.value))
    S._inner = Ah
    S.validate()


def test_march_says_why_it_was_declined(tf):
    """tf_schedule_info.march_declined: marching runs need N % 64 == 0, rows of at most 32 entries in both
    patterns and a grid; a schedule without them says which of these was missing."""
    A = tf.workloads.laplacian_3d(12)
    Ah = tf.CsrMatrix.from_scipy(A)
    built = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Ah).info()
    assert built["marched"] == 1 and built["march_declined"] == 0           # TF_MARCH_BUILT
    assert tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64).info()["march_declined"] == 1            # no inner pattern: not tried
    assert tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Ah, march=-1).info()["march_declined"] == 1
    assert tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=32, inner=Ah).info()["march_declined"] == 2  # N % 64
    # a 27-point stencil (rows of up to 27 entries) marches, with ELL rows of 32 pairs; a stencil that reaches two
    # points each way (125 points) has rows of more than 32 entries
    e = np.ones(12)
    t = sp.diags([e[:-1], e, e[:-1]], [-1, 0, 1])
    t2 = sp.diags([e[:-2], e[:-1], e, e[:-1], e[:-2]], [-2, -1, 0, 1, 2])

    def box(t):
        W = sp.csr_matrix(sp.kron(sp.kron(t, t), t), dtype=np.float32)
        W.sort_indices()
        return sp.csr_matrix((W.data, W.indices.astype(np.int32), W.indptr.astype(np.int32)), shape=W.shape)
    W27h = tf.CsrMatrix.from_scipy(box(t))
    S27 = tf.inspector(W27h, 1, op=tf.OP_SPMM_SPMM, N=64, inner=W27h)
    S27.validate()
    assert S27.info()["marched"] == 1 and S27.info()["march_declined"] == 0
    Wh = tf.CsrMatrix.from_scipy(box(t2))
    assert tf.inspector(Wh, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Wh).info()["march_declined"] == 3
    # short rows, but no grid to be found and none given; a grid that does not multiply to the row count
    R = tf.workloads.erdos_renyi_gcn(1500, 2.0, seed=4)
    R = sp.csr_matrix(R.multiply(sp.csr_matrix(np.diff(R.indptr)[:, None] <= 8)), dtype=np.float32)
    deg = np.diff(R.indptr)
    if deg.max() <= 8:
        R.sort_indices()
        R = sp.csr_matrix((R.data, R.indices.astype(np.int32), R.indptr.astype(np.int32)), shape=R.shape)
        Rh = tf.CsrMatrix.from_scipy(R)
        assert tf.inspector(Rh, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Rh).info()["march_declined"] == 4
    assert tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Ah, grid=(12, 12, 11)).info()["march_declined"] == 4
    with pytest.raises(tf.TileFusionError):
        tf.inspector(Wh, 1, op=tf.OP_SPMM_SPMM, N=64, inner=Wh, march=1)


def test_short_rows_mark_their_cold_gathers_on_power_law_graphs(tf):
    """short_row_hot_bytes: on a graph with hub rows (long rows column-partitioned) the short remainder rows keep
    their gathers of the most-read intermediate rows cacheable and mark all others as streaming; a graph without
    a hot set (Erdos-Renyi) marks nothing; the schedule validates either way and -1 switches it off."""
    cfg = tf.workloads.make_config(4, 2.0 ** -5)
    Ah = tf.CsrMatrix.from_scipy(cfg["A"])
    S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128, long_row_partition=1)
    S.validate()
    info = S.info()
    assert info["long_row_hot_cols"] > 0 and 0 < info["short_row_hot_rows"] <= (32 << 20) // 512
    S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128, long_row_partition=1, short_row_hot_bytes=1 << 20)
    S.validate()
    assert 0 < S.info()["short_row_hot_rows"] <= 2048
    assert tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128, long_row_partition=1, short_row_hot_bytes=-1).info()["short_row_hot_rows"] == 0
    er = tf.workloads.make_config(3, 0.05)
    Eh = tf.CsrMatrix.from_scipy(er["A"])
    S = tf.inspector(Eh, 1, op=tf.OP_GEMM_SPMM, N=128, K=256, short_row_hot_bytes=256 << 10)   # 512 of 10,000 rows
    S.validate()
    assert S.info()["short_row_hot_rows"] == 0


def test_intermediate_rows_are_placed_where_nothing_fuses(tf):
    """place_intermediate: a GeMM-SpMM schedule in which nothing fuses and every gather goes through the schedule's own
    lists (a power-law graph, an Erdos-Renyi graph) stores the intermediate's rows in the order they are read most;
    the validator checks the lists against the places.  Schedules with fused tiles (a band), SpMM-SpMM schedules and
    -1 leave the rows at their own index."""
    cfg = tf.workloads.make_config(4, 2.0 ** -5)
    Ah = tf.CsrMatrix.from_scipy(cfg["A"])
    S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128, long_row_partition=1)
    S.validate()
    assert S.info()["intermediate_placed"] == 1 and S.info()["n_fused_rows"] == 0
    S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128, long_row_partition=1, place_intermediate=-1)
    S.validate()
    assert S.info()["intermediate_placed"] == 0
    # long rows in chunks (no column partition at this size) read A's own columns: nothing placed
    S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=128, K=128)
    S.validate()
    assert S.info()["n_long_chunks"] > 0 and S.info()["intermediate_placed"] == 0
    er = tf.workloads.make_config(3, 0.05)
    Eh = tf.CsrMatrix.from_scipy(er["A"])
    S = tf.inspector(Eh, 1, op=tf.OP_GEMM_SPMM, N=128, K=256)
    S.validate()
    assert S.info()["intermediate_placed"] == 1
    # the rows of the list read A in place (reorder_adjacency = -1): nothing to translate, nothing placed
    S = tf.inspector(Eh, 1, op=tf.OP_GEMM_SPMM, N=128, K=256, reorder_adjacency=-1)
    S.validate()
    assert S.info()["intermediate_placed"] == 0
    band = tf.workloads.banded_random(30000, 32, 12, seed=3)
    Bh = tf.CsrMatrix.from_scipy(band)
    S = tf.inspector(Bh, 1, op=tf.OP_GEMM_SPMM, N=128, K=128)
    S.validate()
    assert S.info()["n_fused_rows"] > 0 and S.info()["intermediate_placed"] == 0
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=128)
    S.validate()
    assert S.info()["intermediate_placed"] == 0


# ---- two-layer tiles -------------------------------------------------------------------------------------------

def _check_two_layer_tiles(A, rng6, H, N):
    """Independent of the library: owned ranges partition the rows in order; every owned row reads hidden rows of
    its tile only, every hidden row of the tile rows of the first intermediate the tile computes; slabs fit LDS."""
    M = A.shape[0]
    end = 0
    for o0, o1, h0, h1, t0, t1 in rng6:
        assert o0 == end and o1 > o0
        end = o1
        cols = A.indices[A.indptr[o0]:A.indptr[o1]]
        if len(cols):
            assert cols.min() >= h0 and cols.max() < h1
        hc = A.indices[A.indptr[h0]:A.indptr[h1]] if h1 > h0 else np.zeros(0, int)
        if len(hc):
            assert hc.min() >= t0 and hc.max() < t1
        a = max((t1 - t0) * (H + 4), (h1 - h0) * (N + 4))
        b = max((h1 - h0) * (H + 4), 2 * 64 * 36)
        c0, c1 = (min(o0, h0), max(o1, h1)) if h1 > h0 else (o0, o1)   # the tile's copy of A's rows
        al = lambda x: (x + 3) // 4 * 4  # noqa: E731
        c = al(c1 - c0 + 1) + 2 * al(int(A.indptr[c1] - A.indptr[c0]))
        assert (a + b + c) * 4 <= 163840
    assert end == M


def test_two_layer_tiles_on_banded_patterns(tf):
    """GeMM-SpMM schedules of a banded matrix carry two-layer tiles (what tf_gcn_two_layers runs when the schedule
    is its second layer's): exact ranges on a band of half-width 16, for the widths the kernel is built for; the
    library's validator and an independent one agree; patterns without a band, other widths and the opt-out get none."""
    M = 6000
    A = tf.workloads.banded_random(M, 32, 16, seed=3)
    for H, N in ((128, 128), (64, 64), (128, 64), (32, 128)):
        S, view, info = inspect(tf, A, op=tf.OP_GEMM_SPMM, N=N, K=H, compute_units=16)
        assert info["two_layer_tiles"] > 0 and len(view["two_layer_range"]) == info["two_layer_tiles"]
        _check_two_layer_tiles(A, view["two_layer_range"], H, N)
        r = view["two_layer_range"]
        inner = r[1:-1]
        # a band of half-width 16: hidden halo of at most 16 rows a side, the first intermediate's 16 more
        assert np.all(inner[:, 0] - inner[:, 2] <= 16) and np.all(inner[:, 3] - inner[:, 1] <= 16)
        assert np.all(inner[:, 2] - inner[:, 4] <= 16) and np.all(inner[:, 5] - inner[:, 3] <= 16)
        assert np.all(inner[:, 1] - inner[:, 0] >= 32)
    # widths the kernel is not built for, the opt-out, a pattern whose halos no LDS holds
    assert inspect(tf, A, op=tf.OP_GEMM_SPMM, N=96, K=128)[2]["two_layer_tiles"] == 0
    assert inspect(tf, A, op=tf.OP_GEMM_SPMM, N=128, K=40)[2]["two_layer_tiles"] == 0
    assert inspect(tf, A, op=tf.OP_GEMM_SPMM, N=7, K=64)[2]["two_layer_tiles"] == 0    # (runs as a padded panel of 32 columns)
    assert inspect(tf, A, op=tf.OP_GEMM_SPMM, N=30, K=64)[2]["two_layer_tiles"] == 0
    assert inspect(tf, A, op=tf.OP_GEMM_SPMM, N=128, K=128, two_layer_tiles=-1)[2]["two_layer_tiles"] == 0
    er = tf.workloads.make_config(3, 0.05)["A"]
    assert inspect(tf, er, op=tf.OP_GEMM_SPMM, N=128, K=128)[2]["two_layer_tiles"] == 0
    # rows without entries, and a 2D grid (halo of a grid line a side)
    L2 = tf.workloads.laplacian_2d(40)
    S, view, info = inspect(tf, L2, op=tf.OP_GEMM_SPMM, N=64, K=64, compute_units=8)
    assert info["two_layer_tiles"] > 0
    _check_two_layer_tiles(L2, view["two_layer_range"], 64, 64)
    E = sp.csr_matrix(sp.diags(np.r_[np.zeros(300), np.ones(M - 300)].astype(np.float32)) @ A)
    E.eliminate_zeros(); E.sort_indices()
    E = sp.csr_matrix((E.data.astype(np.float32), E.indices.astype(np.int32), E.indptr.astype(np.int32)), shape=E.shape)
    S, view, info = inspect(tf, E, op=tf.OP_GEMM_SPMM, N=64, K=64, compute_units=16)
    assert info["two_layer_tiles"] > 0
    _check_two_layer_tiles(E, view["two_layer_range"], 64, 64)


def test_two_layer_tiles_are_validated_against_the_pattern(tf):
    """The validator replays the two-layer tiles too: a pattern with one column moved out of a tile's halo is refused."""
    M = 3000
    A = tf.workloads.banded_random(M, 32, 16, seed=3)
    Ah = tf.CsrMatrix.from_scipy(A)
    S = tf.inspector(Ah, 1, op=tf.OP_GEMM_SPMM, N=64, K=64, compute_units=16, lds_budget_bytes=163840, tile_rows=3000, max_redundancy=1.0)
    assert S.info()["two_layer_tiles"] > 1
    S.validate()
    r = S.view()["two_layer_range"]
    o0, o1, h0, h1, t0, t1 = r[1]
    B = A.copy(); B.indices = B.indices.copy()
    row = (o0 + o1) // 2
    B.indices[B.indptr[row]] = max(0, h0 - 40)          # an owned row now reads a hidden row the tile does not compute
    B.has_sorted_indices = False
    with pytest.raises(tf.TileFusionError) as e:
        S.validate(tf.CsrMatrix.from_scipy(B))
    assert e.value.status == -4


def _random_band(M, lo_off, hi_off, per_row, seed, empty_share=0.0):
    """Row i holds up to per_row distinct columns drawn from [i + lo_off, i + hi_off] clipped to the matrix."""
    rng = np.random.default_rng(seed)
    rows, cols = [], []
    for i in range(M):
        if rng.random() < empty_share:
            continue
        a, b = max(0, i + lo_off), min(M - 1, i + hi_off)
        if a > b:
            continue
        c = np.unique(rng.integers(a, b + 1, per_row))
        rows += [i] * len(c)
        cols += c.tolist()
    A = sp.csr_matrix((rng.uniform(-1, 1, len(rows)).astype(np.float32), (rows, cols)), shape=(M, M))
    A.sort_indices()
    return sp.csr_matrix((A.data, A.indices.astype(np.int32), A.indptr.astype(np.int32)), shape=A.shape)


@pytest.mark.parametrize("lo_off,hi_off,per_row,empty", [(-16, 15, 16, 0.0), (-40, -1, 6, 0.0), (1, 30, 5, 0.1), (-3, 3, 7, 0.3),
                                                         (-200, -150, 4, 0.0), (-64, 64, 40, 0.05)])
def test_two_layer_tiles_on_irregular_bands(tf, lo_off, hi_off, per_row, empty):
    """Bands that do not hold the diagonal (strictly lower, strictly upper, far off it), rows without entries, rows of
    many entries: the owned rows of a tile then need not lie inside its hidden range, and the tile's copy of A's rows
    spans both.  Every schedule with tiles passes the library's validator and the independent check."""
    M = 5000
    A = _random_band(M, lo_off, hi_off, per_row, seed=11, empty_share=empty)
    for H, N in ((64, 64), (128, 32)):
        S, view, info = inspect(tf, A, op=tf.OP_GEMM_SPMM, N=N, K=H, compute_units=16)
        if info["two_layer_tiles"]:
            _check_two_layer_tiles(A, view["two_layer_range"], H, N)
        else:                                  # no tiles only if some single row's two halos and its rows of A exceed LDS
            def alone(i):
                cols = A.indices[A.indptr[i]:A.indptr[i + 1]]
                if not len(cols):
                    return 0
                h0, h1 = cols.min(), cols.max() + 1
                hc = A.indices[A.indptr[h0]:A.indptr[h1]]
                t0, t1 = (hc.min(), hc.max() + 1) if len(hc) else (0, 0)
                c0, c1 = min(i, h0), max(i + 1, h1)
                al = lambda x: (x + 3) // 4 * 4  # noqa: E731
                return (max((t1 - t0) * (H + 4), (h1 - h0) * (N + 4)) + max((h1 - h0) * (H + 4), 2 * 64 * 36)
                        + al(c1 - c0 + 1) + 2 * al(int(A.indptr[c1] - A.indptr[c0]))) * 4
            assert max(alone(i) for i in range(M)) > 163840
