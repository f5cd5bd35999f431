"""ctypes doors onto the checker: oracle/liboracle.so (the C restatement) and, when it has
been built, oracle/_ref/libtf_ref.so (the reference's own translation units).  Test
infrastructure only; nothing in the product imports this."""
import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_SO = os.path.join(ROOT, "oracle", "liboracle.so")
REF_SO = os.path.join(ROOT, "oracle", "_ref", "libtf_ref.so")

_PI = C.POINTER(C.c_int)
_PF = C.POINTER(C.c_float)


class OrcSchedule(C.Structure):
    _fields_ = [("n1", C.c_int), ("n_part", C.c_int), ("n_id", C.c_int), ("ptr1", _PI), ("ptr2", _PI),
                ("ker_begin", _PI), ("id", _PI), ("type", _PI)]


_orc = None
_ref = None


def oracle():
    global _orc
    if _orc is None:
        if not os.path.exists(ORACLE_SO):
            raise ImportError(f"{ORACLE_SO} missing: run `make -C oracle`")
        _orc = C.CDLL(ORACLE_SO)
        _orc.orc_max_threads.restype = C.c_int
    return _orc


def ref():
    """The compiled reference units, or None when they were not built / cannot run here."""
    global _ref
    if _ref is None:
        if not os.path.exists(REF_SO):
            return None
        lib = C.CDLL(REF_SO)
        lib.ref_cpu_ok.restype = C.c_int
        if not lib.ref_cpu_ok():
            return None
        _ref = lib
    return _ref


def _i(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def pi(a):
    return a.ctypes.data_as(_PI)


def pf(a):
    return a.ctypes.data_as(_PF)


def max_threads():
    return int(oracle().orc_max_threads())


class Schedule:
    """Numpy copies of a MultiDimensionalSet-layout schedule."""

    def __init__(self, n1, ptr1, ptr2, ker_begin, ids, types):
        self.n1 = int(n1)
        self.ptr1, self.ptr2, self.ker_begin, self.id, self.type = map(_i, (ptr1, ptr2, ker_begin, ids, types))

    @classmethod
    def from_struct(cls, s):
        P, n = s.n_part, s.n_id
        g = lambda p, k: np.ctypeslib.as_array(p, shape=(k,)).copy() if k > 0 else np.zeros(0, np.int32)
        out = cls(s.n1, g(s.ptr1, 3), g(s.ptr2, P + 1), g(s.ker_begin, 2 * P), g(s.id, n), g(s.type, n))
        oracle().orc_schedule_free(C.byref(s))
        return out

    @property
    def n_tiles(self):
        return int(self.ptr1[1])

    def tiles(self):
        """[(first_op_rows, fused_second_op_rows)] for level 0, [rows] for level 1."""
        lvl0 = []
        for p in range(self.ptr1[0], self.ptr1[1]):
            lvl0.append((self.id[self.ptr2[p]:self.ker_begin[2 * p]], self.id[self.ker_begin[2 * p]:self.ker_begin[2 * p + 1]]))
        lvl1 = [self.id[self.ptr2[p]:self.ptr2[p + 1]] for p in range(self.ptr1[1], self.ptr1[self.n1] if self.n1 > 1 else self.ptr1[1])]
        return lvl0, lvl1


def inspect_vt_gemm_spmm(A, BCol, CCol, cache_bytes, data_size=4):
    s = OrcSchedule()
    ap, ai = _i(A.indptr), _i(A.indices)
    rc = oracle().orc_inspect_vt_gemm_spmm(A.shape[0], A.shape[1], pi(ap), pi(ai), BCol, CCol, cache_bytes, data_size, C.byref(s))
    if rc:
        raise ValueError(f"orc_inspect_vt_gemm_spmm failed: {rc}")
    return Schedule.from_struct(s)


def inspect_vt_both_wavefronts(A, BCol, cache_bytes, num_threads, data_size=4):
    s = OrcSchedule()
    ap, ai = _i(A.indptr), _i(A.indices)
    rc = oracle().orc_inspect_vt_both_wavefronts(A.shape[0], A.shape[1], pi(ap), pi(ai), BCol, cache_bytes, data_size, num_threads, C.byref(s))
    if rc:
        raise ValueError(f"orc_inspect_vt_both_wavefronts failed: {rc}")
    return Schedule.from_struct(s)


def inspect_fixed_tiles(A, iter_per_partition, num_threads):
    s = OrcSchedule()
    ap, ai = _i(A.indptr), _i(A.indices)
    rc = oracle().orc_inspect_fixed_tiles(A.shape[0], pi(ap), pi(ai), iter_per_partition, num_threads, C.byref(s))
    if rc:
        raise ValueError(f"orc_inspect_fixed_tiles failed: {rc}")
    return Schedule.from_struct(s)


def unfused_schedule(M, rows_per_part=64):
    """Two levels without any fusion: level 0 = all first-op rows, level 1 = all second-op rows."""
    nparts = (M + rows_per_part - 1) // rows_per_part
    bounds = np.minimum(np.arange(nparts + 1) * rows_per_part, M).astype(np.int32)
    ids = np.concatenate([np.arange(M), np.arange(M)]).astype(np.int32)
    types = np.concatenate([np.zeros(M), np.ones(M)]).astype(np.int32)
    ptr2 = np.concatenate([bounds, M + bounds[1:]]).astype(np.int32)
    kb = np.empty(4 * nparts, np.int32)
    kb[0:2 * nparts:2] = bounds[1:]
    kb[1:2 * nparts:2] = bounds[1:]
    kb[2 * nparts::2] = M + bounds[:-1]
    kb[2 * nparts + 1::2] = M + bounds[1:]
    return Schedule(2, [0, nparts, 2 * nparts], ptr2, kb, ids, types)


def spmm(A, X, nthreads=1):
    M, N = A.shape[0], X.shape[1]
    ap, ai, ax, x = _i(A.indptr), _i(A.indices), _f(A.data), _f(X)
    out = np.zeros((M, N), np.float32)
    oracle().orc_spmm_csr(M, N, pi(ap), pi(ai), pf(ax), pf(x), pf(out), nthreads)
    return out


def ref_spmm(A, X, nthreads=1):
    """Y = A*X by the reference's own spmmCsrParallel<float> (fusion/src/SpMM_SpMM.cpp:37-55)."""
    M, N = A.shape[0], X.shape[1]
    ap, ai, ax, x = _i(A.indptr), _i(A.indices), _f(A.data), _f(X)
    out = np.zeros((M, N), np.float32)
    ref().ref_spmm_csr_parallel(M, N, A.shape[1], pi(ap), pi(ai), pf(ax), pf(x), pf(out), nthreads)
    return out


def spmm_spmm(A, B, Cd, sched, nthreads=1, impl="oracle"):
    """D = A*(B*C) (README naming) over an interleaved schedule.  impl: 'oracle' |
    'ref_scalar' | 'ref_vec32' (the last two run the reference's compiled code)."""
    L, M, N = A.shape[0], B.shape[0], Cd.shape[1]
    ap, ai, ax = _i(A.indptr), _i(A.indices), _f(A.data)
    bp, bi, bx = _i(B.indptr), _i(B.indices), _f(B.data)
    c = _f(Cd)
    D = np.zeros((L, N), np.float32)
    T = np.zeros((M, N), np.float32)
    # reference argument order: inner matrix first ("A" there), outer second ("B" there)
    if impl == "oracle":
        oracle().orc_spmm_spmm_fused(M, N, pi(bp), pi(bi), pf(bx), pi(ap), pi(ai), pf(ax), pf(c), pf(D), pf(T),
                                     sched.n1, pi(sched.ptr1), pi(sched.ptr2), pi(sched.id), pi(sched.type), nthreads)
    else:
        fn = {"ref_scalar": ref().ref_spmm_spmm_fused_scalar, "ref_vec32": ref().ref_spmm_spmm_fused_vec32}[impl]
        fn(M, N, B.shape[1], L, pi(bp), pi(bi), pf(bx), pi(ap), pi(ai), pf(ax), pf(c), pf(D), pf(T),
           sched.n1, pi(sched.ptr1), pi(sched.ptr2), pi(sched.id), pi(sched.type), nthreads)
    return D, T


def spmm_spmm_separated(A, Cd, sched, nthreads=1, impl="oracle"):
    """D = A*(A*C) over the separated walk (one sparse matrix)."""
    M, N = A.shape[0], Cd.shape[1]
    ap, ai, ax, c = _i(A.indptr), _i(A.indices), _f(A.data), _f(Cd)
    D = np.zeros((M, N), np.float32)
    T = np.zeros((M, N), np.float32)
    if impl == "oracle":
        oracle().orc_spmm_spmm_fused_separated(M, N, pi(ap), pi(ai), pf(ax), pf(c), pf(D), pf(T), sched.n1,
                                               pi(sched.ptr1), pi(sched.ptr2), pi(sched.id), pi(sched.ker_begin), nthreads)
    else:
        ref().ref_spmm_spmm_fused_separated_vec32(M, N, M, M, pi(ap), pi(ai), pf(ax), pf(c), pf(D), pf(T), sched.n1,
                                                  pi(sched.ptr1), pi(sched.ptr2), pi(sched.id), pi(sched.ker_begin), nthreads)
    return D, T


def simd():
    """1 when the oracle's GEMM runs its AVX-512 body on this host."""
    o = oracle()
    o.orc_simd.restype = C.c_int
    return int(o.orc_simd())


def set_simd(on):
    """False forces the scalar body of the oracle's GEMM (the two give the same bits)."""
    oracle().orc_set_simd(1 if on else 0)


def gemm(X, W, nthreads=1):
    M, K = X.shape
    N = W.shape[1]
    x, w = _f(X), _f(W)
    out = np.zeros((M, N), np.float32)
    oracle().orc_sgemm(M, N, K, pf(x), pf(w), pf(out), nthreads)
    return out


def gemm_spmm(A, B, Cd, sched, nthreads=1):
    """D = A*(B*C), B and C dense, over the separated walk."""
    M, K = B.shape
    N = Cd.shape[1]
    ap, ai, ax = _i(A.indptr), _i(A.indices), _f(A.data)
    b, c = _f(B), _f(Cd)
    D = np.zeros((A.shape[0], N), np.float32)
    T = np.zeros((M, N), np.float32)
    oracle().orc_gemm_spmm_fused(M, pi(ap), pi(ai), pf(ax), K, N, pf(b), pf(c), pf(D), pf(T), nthreads, sched.n1,
                                 pi(sched.ptr1), pi(sched.ptr2), pi(sched.ker_begin), pi(sched.id))
    return D, T


def rel_err(got, want):
    """max |got - want| / max |want| : the error measure of the 1e-4 gate."""
    want = np.asarray(want, dtype=np.float64)
    scale = max(float(np.abs(want).max()), 1e-30)
    return float(np.abs(np.asarray(got, dtype=np.float64) - want).max() / scale)
