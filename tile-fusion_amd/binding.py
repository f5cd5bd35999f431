"""ctypes binding of libtilefusion_hip (declared in include/tilefusion_hip.h).

Mirrors the README API of the reference (README.md:21-38): ``inspector`` builds a
``FusedSchedule`` from a CSR matrix, ``spmm_spmm`` / ``gemm_spmm`` are the executors.
There is no fallback: if the shared library is missing, loading raises.
"""
import ctypes as C
import os

import numpy as np

OP_SPMM_SPMM = 0
OP_GEMM_SPMM = 1
ACCUMULATE = 1
SECOND_STREAM = 2
RELU = 4
FUSE_LAYERS = 8

_HERE = os.path.dirname(os.path.abspath(__file__))


def lib_path():
    return os.path.join(_HERE, "lib", "libtilefusion_hip.so")


class TileFusionError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"tilefusion status {status}: {message}")
        self.status = status


class DeviceInfo(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("device", C.c_int), ("compute_units", C.c_int), ("xcds", C.c_int),
                ("lds_bytes_per_block", C.c_int), ("wavefront", C.c_int), ("clock_khz", C.c_int),
                ("hbm_bytes", C.c_size_t), ("arch", C.c_char * 64), ("xcd_round_robin", C.c_int)]


class InspectOpts(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("op", C.c_int), ("N", C.c_int), ("K", C.c_int), ("lds_budget_bytes", C.c_int),
                ("tile_rows", C.c_int), ("max_redundancy", C.c_float), ("long_row_nnz", C.c_int),
                ("compute_units", C.c_int), ("inner_Ap", C.POINTER(C.c_int)), ("inner_Ai", C.POINTER(C.c_int)),
                ("inner_cols", C.c_int), ("strip_cols", C.c_int), ("xcd_chunk_rows", C.c_int), ("wide_strips", C.c_int), ("long_row_partition", C.c_int),
                ("march", C.c_int), ("grid_nx", C.c_int), ("grid_ny", C.c_int), ("grid_nz", C.c_int),
                ("march_tile_x", C.c_int), ("march_tile_y", C.c_int), ("reorder_adjacency", C.c_int), ("hot_partition_bytes", C.c_int),
                ("short_row_hot_bytes", C.c_int), ("two_layer_tiles", C.c_int), ("place_intermediate", C.c_int)]


class ScheduleInfo(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("op", C.c_int), ("N", C.c_int), ("K", C.c_int), ("rows", C.c_int),
                ("inter_rows", C.c_int), ("n_tiles", C.c_int), ("n_fused_rows", C.c_int),
                ("n_remainder_rows", C.c_int), ("n_long_rows", C.c_int), ("n_long_chunks", C.c_int),
                ("n_producer_rows", C.c_int), ("n_writeback_rows", C.c_int),
                ("max_tile_producer_rows", C.c_int), ("lds_bytes", C.c_int), ("windowed", C.c_int),
                ("strip_cols", C.c_int), ("xcd_chunk_rows", C.c_int), ("streamed", C.c_int), ("ring_rows", C.c_int), ("wide_strips", C.c_int), ("long_row_hot_cols", C.c_int),
                ("fused_nnz", C.c_longlong), ("workspace_bytes", C.c_longlong),
                ("marched", C.c_int), ("march_tile_x", C.c_int), ("march_tile_y", C.c_int), ("march_slots", C.c_int),
                ("march_declined", C.c_int), ("register_weights", C.c_int), ("n_zero_rows", C.c_int), ("two_layer_tiles", C.c_int),
                ("short_row_hot_rows", C.c_int), ("n_computed_rows", C.c_int), ("intermediate_placed", C.c_int)]


class ScheduleView(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("n1", C.c_int), ("n_part", C.c_int), ("n_id", C.c_int), ("n_tiles", C.c_int),
                ("ptr1", C.POINTER(C.c_int)), ("ptr2", C.POINTER(C.c_int)),
                ("ker_begin", C.POINTER(C.c_int)), ("id", C.POINTER(C.c_int)),
                ("type", C.POINTER(C.c_int)), ("tile_range", C.POINTER(C.c_int)),
                ("writeback", C.POINTER(C.c_int)), ("tile_step", C.POINTER(C.c_int)),
                ("step_ptr", C.POINTER(C.c_int)), ("n_step_ptr", C.c_int),
                ("two_layer_range", C.POINTER(C.c_int)), ("n_two_layer", C.c_int)]


PROFILE_MAX = 16


class Profile(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("n", C.c_int), ("name", C.c_char_p * PROFILE_MAX), ("ms", C.c_float * PROFILE_MAX)]


_PI = C.POINTER(C.c_int)
_PF = C.POINTER(C.c_float)
_VP = C.c_void_p

# name -> (restype, argtypes); every symbol include/tilefusion_hip.h declares
SIGNATURES = {
    "tf_last_error_string": (C.c_char_p, []),
    "tf_version": (C.c_char_p, []),
    "tf_device_init": (C.c_int, [C.c_int, C.POINTER(DeviceInfo)]),
    "tf_device_synchronize": (C.c_int, []),
    "tf_stream_create": (C.c_int, [C.POINTER(_VP)]),
    "tf_stream_destroy": (C.c_int, [_VP]),
    "tf_stream_synchronize": (C.c_int, [_VP]),
    "tf_event_create": (C.c_int, [C.POINTER(_VP)]),
    "tf_event_destroy": (C.c_int, [_VP]),
    "tf_event_record": (C.c_int, [_VP, _VP]),
    "tf_event_synchronize": (C.c_int, [_VP]),
    "tf_event_elapsed_ms": (C.c_int, [_VP, _VP, _PF]),
    "tf_csr_upload": (C.c_int, [C.c_int, C.c_int, _PI, _PI, _PF, C.POINTER(_VP)]),
    "tf_csr_wrap_device": (C.c_int, [C.c_int, C.c_int, C.c_int, _VP, _VP, _VP, C.POINTER(_VP)]),
    "tf_pattern_hash": (C.c_uint64, [C.c_int, _PI, _PI]),
    "tf_csr_set_pattern_hash": (C.c_int, [_VP, C.c_uint64]),
    "tf_csr_free": (None, [_VP]),
    "tf_dense_upload": (C.c_int, [C.c_int, C.c_int, _PF, C.POINTER(_VP)]),
    "tf_dense_alloc": (C.c_int, [C.c_int, C.c_int, C.POINTER(_VP)]),
    "tf_dense_wrap_device": (C.c_int, [C.c_int, C.c_int, _VP, C.POINTER(_VP)]),
    "tf_dense_download": (C.c_int, [_VP, _PF]),
    "tf_dense_fill": (C.c_int, [_VP, C.c_float, _VP]),
    "tf_dense_copy": (C.c_int, [_VP, _VP, _VP]),
    "tf_dense_device_ptr": (_VP, [_VP]),
    "tf_dense_free": (None, [_VP]),
    "tf_read_matrix": (C.c_int, [C.c_char_p, _PI, _PI, _PI, C.POINTER(_PI), C.POINTER(_PI), C.POINTER(_PF)]),
    "tf_read_dense": (C.c_int, [C.c_char_p, _PI, _PI, C.POINTER(_PF)]),
    "tf_host_free": (None, [_VP]),
    "tf_reorder_rcm": (C.c_int, [C.c_int, _PI, _PI, _PI]),
    "tf_reorder_partition": (C.c_int, [C.c_int, _PI, _PI, C.c_int, C.c_int, _PI, _PI]),
    "tf_permute_csr": (C.c_int, [C.c_int, _PI, _PI, _PF, _PI, C.POINTER(_PI), C.POINTER(_PI), C.POINTER(_PF)]),
    "tf_inspect": (C.c_int, [C.c_int, C.c_int, _PI, _PI, C.POINTER(InspectOpts), C.POINTER(_VP)]),
    "tf_schedule_free": (None, [_VP]),
    "tf_schedule_get_info": (C.c_int, [_VP, C.POINTER(ScheduleInfo)]),
    "tf_schedule_get_view": (C.c_int, [_VP, C.POINTER(ScheduleView)]),
    "tf_schedule_validate": (C.c_int, [_VP, C.c_int, C.c_int, _PI, _PI]),
    "tf_schedule_validate_inner": (C.c_int, [_VP, C.c_int, C.c_int, _PI, _PI, _PI, _PI, C.c_int]),
    "tf_schedule_set_profiling": (C.c_int, [_VP, C.c_int]),
    "tf_schedule_get_profile": (C.c_int, [_VP, C.POINTER(Profile)]),
    "tf_spmm_spmm_noalloc": (C.c_int, [_VP, _VP, _VP, _VP, C.c_uint, _VP]),
    "tf_noalloc_scratch_bytes": (C.c_size_t, []),
    "tf_spmm_spmm": (C.c_int, [_VP, _VP, _VP, _VP, _VP, C.c_uint, _VP]),
    "tf_gemm_spmm": (C.c_int, [_VP, _VP, _VP, _VP, _VP, C.c_uint, _VP]),
    "tf_gcn_two_layers": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, C.c_uint, _VP]),
    "tf_spmm": (C.c_int, [_VP, _VP, _VP, C.c_uint, _VP]),
    "tf_gemm": (C.c_int, [_VP, _VP, _VP, _VP]),
    "tf_calibrate_issue": (C.c_int, [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_float)]),
}

_lib = None


def lib():
    """The loaded library; raises if it has not been built (no CPU fallback exists)."""
    global _lib
    if _lib is None:
        path = lib_path()
        if not os.path.exists(path):
            raise ImportError(f"{path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`")
        handle = C.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def _check(status):
    if status != 0:
        raise TileFusionError(status, lib().tf_last_error_string().decode())


def _i32(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a, a.ctypes.data_as(_PI)


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_PF)


def device_init(device=0):
    info = DeviceInfo(C.sizeof(DeviceInfo))
    _check(lib().tf_device_init(device, C.byref(info)))
    return {f: (getattr(info, f).decode() if f == "arch" else getattr(info, f)) for f, _ in DeviceInfo._fields_ if f != "struct_size"}


def calibrate_issue(role_older, role_younger, iters=2000):
    """Duration in ms of the issue probe (tf_calibrate_issue): roles 0 nothing, 1 fp32 MFMA, 2 fp32 FMA, 3 bf16 MFMA."""
    ms = C.c_float()
    _check(lib().tf_calibrate_issue(role_older, role_younger, iters, C.byref(ms)))
    return ms.value


def device_synchronize():
    _check(lib().tf_device_synchronize())


class Stream:
    def __init__(self):
        self.h = _VP()
        _check(lib().tf_stream_create(C.byref(self.h)))

    def synchronize(self):
        _check(lib().tf_stream_synchronize(self.h))

    def __del__(self):
        if getattr(self, "h", None):
            lib().tf_stream_destroy(self.h)
            self.h = None


class Event:
    def __init__(self):
        self.h = _VP()
        _check(lib().tf_event_create(C.byref(self.h)))

    def record(self, stream=None):
        _check(lib().tf_event_record(self.h, stream.h if stream else None))

    def synchronize(self):
        _check(lib().tf_event_synchronize(self.h))

    def elapsed_ms(self, stop):
        ms = C.c_float()
        _check(lib().tf_event_elapsed_ms(self.h, stop.h, C.byref(ms)))
        return ms.value

    def __del__(self):
        if getattr(self, "h", None):
            lib().tf_event_destroy(self.h)
            self.h = None


class CsrMatrix:
    """swiftware::def::CSRMatrix(M, N, Ap, Ai, Ax) (README.md:35): host views, plus a
    device-resident copy made by ``to_device``."""

    def __init__(self, M, N, Ap, Ai, Ax):
        self.M, self.N = int(M), int(N)
        self.Ap, self._pp = _i32(Ap)
        self.Ai, self._pi = _i32(Ai)
        self.Ax, self._px = _f32(Ax)
        self.h = None

    @classmethod
    def from_scipy(cls, m):
        m = m.tocsr()
        return cls(m.shape[0], m.shape[1], m.indptr, m.indices, m.data)

    @property
    def nnz(self):
        return int(self.Ap[-1])

    def to_device(self):
        if self.h is None:
            h = _VP()
            _check(lib().tf_csr_upload(self.M, self.N, self._pp, self._pi, self._px, C.byref(h)))
            self.h = h
        return self

    @classmethod
    def wrap_device(cls, host, dAp, dAi, dAx, pattern_hash=0):
        """A matrix whose arrays already live in device memory (tf_csr_wrap_device): `host` is the CsrMatrix
        with the same arrays on the host (kept for its pattern), dAp/dAi/dAx are device addresses.  The
        library neither copies nor owns them, and takes their values as new on every call."""
        self = cls(host.M, host.N, host.Ap, host.Ai, host.Ax)
        h = _VP()
        _check(lib().tf_csr_wrap_device(self.M, self.N, self.nnz, _VP(dAp), _VP(dAi), _VP(dAx), C.byref(h)))
        if pattern_hash:
            _check(lib().tf_csr_set_pattern_hash(h, pattern_hash))
        self.h = h
        return self

    def __del__(self):
        if getattr(self, "h", None):
            lib().tf_csr_free(self.h)
            self.h = None


class DenseMatrix:
    """swiftware::def::Matrix(M, N, Data) (README.md:36) with a device-resident buffer."""

    def __init__(self, M, N, data=None):
        self.M, self.N = int(M), int(N)
        self.h = _VP()
        if data is None:
            _check(lib().tf_dense_alloc(self.M, self.N, C.byref(self.h)))
        else:
            a, p = _f32(data)
            if a.size != self.M * self.N:
                raise ValueError("data size does not match M x N")
            _check(lib().tf_dense_upload(self.M, self.N, p, C.byref(self.h)))

    @classmethod
    def from_numpy(cls, a):
        a = np.asarray(a)
        return cls(a.shape[0], a.shape[1], a)

    @classmethod
    def wrap_device(cls, M, N, device_ptr):
        self = cls.__new__(cls)
        self.M, self.N = int(M), int(N)
        self.h = _VP()
        _check(lib().tf_dense_wrap_device(self.M, self.N, _VP(device_ptr), C.byref(self.h)))
        return self

    def copy_from(self, src, stream=None):
        _check(lib().tf_dense_copy(self.h, src.h, stream.h if stream else None))

    def fill(self, value, stream=None):
        _check(lib().tf_dense_fill(self.h, float(value), stream.h if stream else None))

    def device_ptr(self):
        return lib().tf_dense_device_ptr(self.h)

    def to_numpy(self):
        out = np.empty((self.M, self.N), dtype=np.float32)
        _check(lib().tf_dense_download(self.h, out.ctypes.data_as(_PF)))
        return out

    def __del__(self):
        if getattr(self, "h", None):
            lib().tf_dense_free(self.h)
            self.h = None


class FusedSchedule:
    """swiftware::def::FusedSchedule: owns the schedule; exposes the reference's flat
    arrays (n1_, ptr1_, ptr2_, ker_begin_, id_, type_) plus the tile ranges."""

    def __init__(self, handle, A, inner=None):
        self.h = handle
        self._A = A
        self._inner = inner

    def info(self):
        s = ScheduleInfo(C.sizeof(ScheduleInfo))
        _check(lib().tf_schedule_get_info(self.h, C.byref(s)))
        return {f: getattr(s, f) for f, _ in ScheduleInfo._fields_ if f != "struct_size"}

    def view(self):
        v = ScheduleView(C.sizeof(ScheduleView))
        _check(lib().tf_schedule_get_view(self.h, C.byref(v)))
        P, nid, nt = v.n_part, v.n_id, v.n_tiles

        def arr(p, n):
            return np.ctypeslib.as_array(p, shape=(n,)).copy() if n > 0 else np.zeros(0, np.int32)
        return {"n1_": v.n1, "ptr1_": arr(v.ptr1, 3), "ptr2_": arr(v.ptr2, P + 1),
                "ker_begin_": arr(v.ker_begin, 2 * P), "id_": arr(v.id, nid), "type_": arr(v.type, nid),
                "tile_range": arr(v.tile_range, 4 * nt).reshape(nt, 4),
                "writeback": arr(v.writeback, 2 * nt).reshape(nt, 2),
                "tile_step": arr(v.tile_step, nt) if v.n_step_ptr else None,
                "step_ptr": arr(v.step_ptr, v.n_step_ptr) if v.n_step_ptr else None,
                "two_layer_range": arr(v.two_layer_range, 8 * v.n_two_layer).reshape(-1, 8)[:, :6] if v.n_two_layer else None}

    def validate(self, A=None):
        """Exact check against the pattern (and the inner pattern, when the schedule was built with one)."""
        A = A or self._A
        B = self._inner
        _check(lib().tf_schedule_validate_inner(self.h, A.M, A.N, A._pp, A._pi, B._pp if B is not None else None,
                                                B._pi if B is not None else None, B.N if B is not None else 0))

    def set_profiling(self, on=True):
        _check(lib().tf_schedule_set_profiling(self.h, 1 if on else 0))

    def profile(self):
        """[(launch name, ms)] of the last executor call with this schedule (profiling switched on)."""
        p = Profile(C.sizeof(Profile))
        _check(lib().tf_schedule_get_profile(self.h, C.byref(p)))
        return [(p.name[i].decode(), float(p.ms[i])) for i in range(p.n)]

    def __del__(self):
        if getattr(self, "h", None):
            lib().tf_schedule_free(self.h)
            self.h = None


def inspector(A, NumThreads=1, *, op, N, K=0, lds_budget_bytes=0, tile_rows=0, max_redundancy=0.0,
              long_row_nnz=0, compute_units=0, inner=None, strip_cols=0, xcd_chunk_rows=0, wide_strips=0, long_row_partition=0,
              march=0, grid=None, march_tile=None, reorder_adjacency=0, hot_partition_bytes=0, short_row_hot_bytes=0, two_layer_tiles=0, place_intermediate=0):
    """swiftware::fusion::inspector(A, NumThreads) (README.md:25).  NumThreads is accepted
    for signature parity and unused: the schedule is sized by the GPU, not by a CPU
    thread count.  The extra keywords are the parameters the reference passes to its
    inspector classes out of band (bCols, embed dim, cache budget).  `inner` is the inner
    sparse matrix B of an SpMM-SpMM (pass A itself when B is A, as in every run of the
    reference); with it the inspector can build windowed tiles."""
    del NumThreads
    o = InspectOpts(C.sizeof(InspectOpts), op, N, K, lds_budget_bytes, tile_rows, max_redundancy, long_row_nnz, compute_units,
                    inner._pp if inner is not None else None, inner._pi if inner is not None else None,
                    inner.N if inner is not None else 0, strip_cols, xcd_chunk_rows, wide_strips, long_row_partition,
                    march, *(grid or (0, 0, 0)), *(march_tile or (0, 0)), reorder_adjacency, hot_partition_bytes, short_row_hot_bytes, two_layer_tiles, place_intermediate)
    h = _VP()
    _check(lib().tf_inspect(A.M, A.N, A._pp, A._pi, C.byref(o), C.byref(h)))
    return FusedSchedule(h, A, inner)


def spmm_spmm(A, B, Cm, D, schedule, NumThreads=1, *, accumulate=False, stream=None, second_stream=False):
    """spMMSpMMExecutor(A, B, C, D, schedule, NumThreads) (README.md:30): D = A*(B*C)."""
    del NumThreads
    _check(lib().tf_spmm_spmm(A.to_device().h, B.to_device().h, Cm.h, D.h, schedule.h,
                              (ACCUMULATE if accumulate else 0) | (SECOND_STREAM if second_stream else 0),
                              stream.h if stream else None))


def gemm_spmm(A, B, Cm, D, schedule, NumThreads=1, *, accumulate=False, stream=None, second_stream=False):
    """geMMSpMMExecutor(A, B, C, D, schedule, NumThreads) (README.md:31): D = A*(B*C)."""
    del NumThreads
    _check(lib().tf_gemm_spmm(A.to_device().h, B.h, Cm.h, D.h, schedule.h,
                              (ACCUMULATE if accumulate else 0) | (SECOND_STREAM if second_stream else 0),
                              stream.h if stream else None))


def gcn_two_layers(A, X, W1, W2, D, s1, s2, *, relu=True, hidden=None, accumulate=False, stream=None, fuse=None):
    """D = A * (act(A * (X * W1)) * W2), the two-layer forward of the reference's end-to-end model
    (binding-project/gcn-e2e-training/FusedGCNModule.py:14-18); the hidden layer stays on the device."""
    _check(lib().tf_gcn_two_layers(A.to_device().h, X.h, W1.h, W2.h, D.h, s1.h, s2.h, hidden.h if hidden is not None else None,
                                   (RELU if relu else 0) | (ACCUMULATE if accumulate else 0) |
                                   (FUSE_LAYERS if fuse else 0), stream.h if stream else None))


def spmm_spmm_noalloc(A, B, Cm, D, *, accumulate=False, stream=None):
    """D = A*(B*C) without a schedule and without any device allocation: the intermediate lives in
    the library's fixed scratch array (see tf_spmm_spmm_noalloc).  A and B must be on the device."""
    if A.h is None or B.h is None:
        raise ValueError("spmm_spmm_noalloc: upload A and B first (to_device allocates)")
    _check(lib().tf_spmm_spmm_noalloc(A.h, B.h, Cm.h, D.h, ACCUMULATE if accumulate else 0, stream.h if stream else None))


def noalloc_scratch_bytes():
    return int(lib().tf_noalloc_scratch_bytes())


def pattern_hash(A):
    """tf_pattern_hash of a scipy CSR matrix or a CsrMatrix."""
    if isinstance(A, CsrMatrix):
        return int(lib().tf_pattern_hash(A.M, A._pp, A._pi))
    ap, ai = _as_i32(A.indptr), _as_i32(A.indices)
    return int(lib().tf_pattern_hash(A.shape[0], ap.ctypes.data_as(_PI), ai.ctypes.data_as(_PI)))


def spmm(A, X, Y, *, accumulate=False, stream=None):
    _check(lib().tf_spmm(A.to_device().h, X.h, Y.h, ACCUMULATE if accumulate else 0,
                         stream.h if stream else None))


def gemm(X, W, Y, *, stream=None):
    _check(lib().tf_gemm(X.h, W.h, Y.h, stream.h if stream else None))


def read_matrix(path):
    """A .mtx / .smtx file as a scipy CSR matrix (int32 indices, fp32 values), read by the
    library's own reader -- the formats the reference's drivers take (Fusion_Utils.cpp:254-272)."""
    import scipy.sparse as sp
    M, N, nnz = C.c_int(), C.c_int(), C.c_int()
    Ap, Ai, Ax = _PI(), _PI(), _PF()
    _check(lib().tf_read_matrix(str(path).encode(), C.byref(M), C.byref(N), C.byref(nnz), C.byref(Ap), C.byref(Ai), C.byref(Ax)))
    try:
        p = np.ctypeslib.as_array(Ap, shape=(M.value + 1,)).copy()
        i = np.ctypeslib.as_array(Ai, shape=(max(nnz.value, 1),))[:nnz.value].copy()
        x = np.ctypeslib.as_array(Ax, shape=(max(nnz.value, 1),))[:nnz.value].copy()
    finally:
        for q in (Ap, Ai, Ax):
            lib().tf_host_free(C.cast(q, _VP))
    return sp.csr_matrix((x, i, p), shape=(M.value, N.value))


def read_dense(path):
    """A MatrixMarket file as a dense row-major fp32 array (Fusion_Utils.cpp:283)."""
    M, N = C.c_int(), C.c_int()
    d = _PF()
    _check(lib().tf_read_dense(str(path).encode(), C.byref(M), C.byref(N), C.byref(d)))
    try:
        out = np.ctypeslib.as_array(d, shape=(max(M.value * N.value, 1),))[:M.value * N.value].copy()
    finally:
        lib().tf_host_free(C.cast(d, _VP))
    return out.reshape(M.value, N.value)


def _as_i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def reorder_rcm(A):
    """Reverse Cuthill-McKee permutation of a square scipy CSR matrix (perm[new] = old), the
    library's counterpart of scipy's reverse_cuthill_mckee in the reference's
    scripts/reorder_graphs.py:21."""
    import scipy.sparse as sp
    A = sp.csr_matrix(A)
    if A.shape[0] != A.shape[1]:
        raise ValueError("reorder_rcm: the matrix must be square")
    M = A.shape[0]
    ap, ai = _as_i32(A.indptr), _as_i32(A.indices)
    perm = np.empty(M, np.int32)
    _check(lib().tf_reorder_rcm(M, ap.ctypes.data_as(_PI), ai.ctypes.data_as(_PI), perm.ctypes.data_as(_PI)))
    return perm


def reorder_partition(A, n_parts, hub_degree=0):
    """Partition-based ordering (tf_reorder_partition): returns (perm, part_ptr) with perm[new] = old; the hubs are
    perm[:part_ptr[1]], part p is perm[part_ptr[p + 1]:part_ptr[p + 2]].  The library's counterpart of the reference's
    graph-partitioner ordering (fusion/src/Fusion_Utils.cpp:181-203)."""
    import scipy.sparse as sp
    A = sp.csr_matrix(A)
    if A.shape[0] != A.shape[1]:
        raise ValueError("reorder_partition: the matrix must be square")
    M = A.shape[0]
    ap, ai = _as_i32(A.indptr), _as_i32(A.indices)
    perm = np.empty(M, np.int32)
    part_ptr = np.zeros(n_parts + 2, np.int32)
    _check(lib().tf_reorder_partition(M, ap.ctypes.data_as(_PI), ai.ctypes.data_as(_PI), int(n_parts), int(hub_degree),
                                      perm.ctypes.data_as(_PI), part_ptr.ctypes.data_as(_PI)))
    return perm, part_ptr


def permute_csr(A, perm):
    """A[perm,:][:,perm] (reorder_graphs.py:22) as a scipy CSR matrix with sorted columns."""
    import scipy.sparse as sp
    A = sp.csr_matrix(A)
    M = A.shape[0]
    ap, ai, ax = _as_i32(A.indptr), _as_i32(A.indices), np.ascontiguousarray(A.data, dtype=np.float32)
    pm = _as_i32(perm)
    if pm.shape != (M,) or A.shape[0] != A.shape[1]:
        raise ValueError("permute_csr: a square matrix and one index per row are needed")
    bp, bi, bx = _PI(), _PI(), _PF()
    _check(lib().tf_permute_csr(M, ap.ctypes.data_as(_PI), ai.ctypes.data_as(_PI), ax.ctypes.data_as(_PF),
                                pm.ctypes.data_as(_PI), C.byref(bp), C.byref(bi), C.byref(bx)))
    try:
        indptr = np.ctypeslib.as_array(bp, shape=(M + 1,)).copy()
        n = int(indptr[M])
        indices = np.ctypeslib.as_array(bi, shape=(max(n, 1),))[:n].copy()
        data = np.ctypeslib.as_array(bx, shape=(max(n, 1),))[:n].copy()
    finally:
        for q in (bp, bi, bx):
            lib().tf_host_free(C.cast(q, _VP))
    return sp.csr_matrix((data, indices, indptr), shape=A.shape)
