"""tf_spmm_spmm_noalloc: D = A*(B*C) for callers that cannot allocate device memory.  Its output
must equal tf_spmm_spmm's bit for bit (and the oracle's), on two calls in a row, the second
with a smaller input -- the fixed scratch array keeps the first call's contents."""
import ctypes as C

import numpy as np
import pytest

from test_gpu_parity import oracle_spmm_spmm, say

pytestmark = pytest.mark.gpu


def _both(tf, A, Cd):
    M, N = A.shape[0], Cd.shape[1]
    Ah = tf.CsrMatrix.from_scipy(A).to_device()
    Cm = tf.DenseMatrix.from_numpy(Cd)
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=N, inner=Ah)
    D1 = tf.DenseMatrix(M, N)
    D1.fill(float("nan"))
    tf.spmm_spmm(Ah, Ah, Cm, D1, S)
    D2 = tf.DenseMatrix(M, N)
    D2.fill(float("nan"))
    tf.spmm_spmm_noalloc(Ah, Ah, Cm, D2)
    tf.device_synchronize()
    return D1.to_numpy(), D2.to_numpy()


def test_noalloc_matches_the_scheduled_executor(gpu, tf, orc):
    say("tf_spmm_spmm_noalloc: two calls, the second smaller")
    assert tf.noalloc_scratch_bytes() == 32 << 20
    # first call fills most of the scratch array, the second uses a part of it
    for M, N, seed in ((60000, 128, 91), (7000, 64, 92)):
        A = tf.workloads.banded_random(M, 32, 16, seed=seed)
        Cd = tf.workloads.uniform((M, N), seed + 10)
        want, got = _both(tf, A, Cd)
        assert np.array_equal(got, want), (M, N)
        assert np.array_equal(got, oracle_spmm_spmm(orc, A, A, Cd)), (M, N)
    # accumulate, two different matrices, rectangular shapes, rows without entries
    L, M, Kc, N = 500, 700, 300, 32
    rng = np.random.default_rng(93)
    import scipy.sparse as sp
    A = sp.random(L, M, density=0.02, random_state=rng, format="csr", dtype=np.float32)
    B = sp.random(M, Kc, density=0.03, random_state=rng, format="csr", dtype=np.float32)
    for m in (A, B):
        m.sort_indices()
        m.indptr, m.indices = m.indptr.astype(np.int32), m.indices.astype(np.int32)
    Cd = tf.workloads.uniform((Kc, N), 94)
    D0 = tf.workloads.uniform((L, N), 95)
    Ah, Bh = tf.CsrMatrix.from_scipy(A).to_device(), tf.CsrMatrix.from_scipy(B).to_device()
    D = tf.DenseMatrix.from_numpy(D0)
    tf.spmm_spmm_noalloc(Ah, Bh, tf.DenseMatrix.from_numpy(Cd), D, accumulate=True)
    T = orc.spmm(B, Cd)
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=N, long_row_nnz=2048)  # every row in CSR order: same bits
    Dref = tf.DenseMatrix.from_numpy(D0)
    tf.spmm_spmm(Ah, Bh, tf.DenseMatrix.from_numpy(Cd), Dref, S, accumulate=True)
    assert np.array_equal(D.to_numpy(), Dref.to_numpy())
    assert orc.rel_err(D.to_numpy(), D0.astype(np.float64) + (A.astype(np.float64) @ T.astype(np.float64))) <= 1e-5


def _hip_runtime():
    """The HIP runtime the library itself is linked against (already loaded into this process)."""
    import ctypes
    with open("/proc/self/maps") as f:
        paths = sorted({line.split()[-1] for line in f if "libamdhip64.so" in line})
    assert paths, "no HIP runtime is loaded"
    return ctypes.CDLL(paths[0])


def _free_device_bytes():
    import ctypes
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert _hip_runtime().hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value   # (of the device: every runtime in the process reports the same)


def test_noalloc_call_allocates_no_device_memory(gpu, tf):
    """What the entry point is for: once the library is initialised on the device (tf_device_init, or one earlier
    call, looks up the scratch array's address) a call leaves the device's free memory exactly as it was -- while
    the probe does see the workspace a scheduled executor allocates on its first call."""
    say("tf_spmm_spmm_noalloc: free device memory unchanged")
    tf.device_init(0)
    M, N = 30000, 64
    A = tf.workloads.erdos_renyi_gcn(M, 8.0, seed=97)         # nothing fuses: a schedule needs the intermediate in HBM
    Ah = tf.CsrMatrix.from_scipy(A).to_device()
    Cm, D = tf.DenseMatrix.from_numpy(tf.workloads.uniform((M, N), 98)), tf.DenseMatrix(M, N)
    st = tf.Stream()
    tf.spmm_spmm_noalloc(Ah, Ah, Cm, D, stream=st)           # warm-up: kernels loaded, address looked up
    st.synchronize()
    tf.device_synchronize()
    free0 = _free_device_bytes()
    for _ in range(3):
        tf.spmm_spmm_noalloc(Ah, Ah, Cm, D, stream=st)
    st.synchronize()
    assert _free_device_bytes() == free0
    # positive control: a scheduled executor's first call allocates its intermediate (30000 x 64 floats = 7.7 MB)
    S = tf.inspector(Ah, 1, op=tf.OP_SPMM_SPMM, N=N)
    assert S.info()["workspace_bytes"] > 4 << 20
    tf.spmm_spmm(Ah, Ah, Cm, D, S, stream=st)
    st.synchronize()
    assert _free_device_bytes() < free0


def test_noalloc_rejects_an_intermediate_beyond_the_scratch(gpu, tf):
    M, N = 70000, 128          # 70,000 x 128 floats = 35.8 MB > 32 MiB
    A = tf.workloads.banded_random(M, 8, 4, seed=96)
    Ah = tf.CsrMatrix.from_scipy(A).to_device()
    Cm, D = tf.DenseMatrix(M, N), tf.DenseMatrix(M, N)
    with pytest.raises(tf.TileFusionError) as e:
        tf.spmm_spmm_noalloc(Ah, Ah, Cm, D)
    assert e.value.status == -5 and "scratch" in str(e.value)


def test_noalloc_call_replays_from_a_graph(gpu, tf, orc):
    """The callers the entry point is for: its two launches are captured into a HIP graph (a capture refuses any
    allocation) and the graph is replayed three times with other values in C, eager work and synchronizations in
    between; every replay equals the eager call and the oracle bit for bit."""
    say("tf_spmm_spmm_noalloc under stream capture")
    hip = _hip_runtime()
    tf.device_init(0)
    M, N = 20000, 64
    A = tf.workloads.banded_random(M, 32, 12, seed=401)
    Ah = tf.CsrMatrix.from_scipy(A).to_device()
    Cs = [tf.workloads.uniform((M, N), 402 + i) for i in range(3)]
    Cm, D = tf.DenseMatrix.from_numpy(Cs[0]), tf.DenseMatrix(M, N)
    st = tf.Stream()
    tf.spmm_spmm_noalloc(Ah, Ah, Cm, D, stream=st)   # eager once: kernels loaded, scratch address looked up
    st.synchronize()
    graph, gexec = C.c_void_p(), C.c_void_p()
    assert hip.hipStreamBeginCapture(st.h, 0) == 0
    try:
        tf.spmm_spmm_noalloc(Ah, Ah, Cm, D, stream=st)
    finally:
        rc = hip.hipStreamEndCapture(st.h, C.byref(graph))
    assert rc == 0 and graph.value
    assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
    try:
        for i in range(3):
            Cm.copy_from(tf.DenseMatrix.from_numpy(Cs[i]), stream=st)
            D.fill(float("nan"), stream=st)
            st.synchronize()
            assert hip.hipGraphLaunch(gexec, st.h) == 0
            st.synchronize()
            got = D.to_numpy()
            assert np.array_equal(got, oracle_spmm_spmm(orc, A, A, Cs[i])), i
    finally:
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)
