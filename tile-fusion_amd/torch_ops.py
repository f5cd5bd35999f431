"""The reference's PyTorch operator surface, ``torch.ops.sw_gcn.*``, on ROCm tensors.

The reference registers these operators from C++ for CPU tensors
(binding-project/main.cpp:133-142) and its Python layers call them
(binding-project/gcn-e2e-training/FusedGCNLayer.py:6-45).  Here the same names, argument
orders and meanings are registered with ``torch.library``; the arithmetic is done by
libtilefusion_hip on the tensors' own device memory (nothing is copied: the CSR arrays and
dense operands are wrapped through ``tf_csr_wrap_device`` / ``tf_dense_wrap_device`` and the
launches go to torch's current stream).  torch is plumbing: it owns the memory and the stream.

    import importlib; importlib.import_module("tile-fusion_amd.torch_ops")
    adj = torch.sparse_csr_tensor(crow.int(), col.int(), val.float(), device="cuda")
    sched = torch.ops.sw_gcn.inspect_vt_ro(adj, in_dim, out_dim, 500000, threads)
    out = torch.ops.sw_gcn.fusedGeMMSpMM_vt_ro(adj, x, weight, sched, threads, 0)   # adj @ (x @ weight.T)

Differences from the reference, all forced by where the data lives:
  * Operands must be ROCm ("cuda") tensors; CPU tensors raise (there is no CPU path here).
    ``inspect`` / ``inspect_vt_ro`` only read the pattern and also accept CPU tensors.
  * The schedule tensors that the inspectors return describe the schedule in the binding
    project's layout (LevelPtr[3]; MixPtr[2p] = start of a partition's first-op ids,
    MixPtr[2p+1] = start of its second-op ids, MixPtr[2P] = end; Partition = the ids;
    Functions.cpp:588-622).  The executors do not parse them back: the native schedule for an
    adjacency and a pair of widths is built once and cached, so any schedule tensors that were
    made for the same adjacency select the same kernels.  MTileSize, CacheSize, NumThreads and
    MaxTileSize are accepted and ignored (tiles are sized by the LDS, not by a CPU cache).
  * Output widths that the MFMA tile GEMM does not take (N % 32, N > 256) are zero-padded or split here;
    the library itself takes any K.
  * The backward pass uses the transpose of the adjacency (the reference multiplies by the
    adjacency itself, Functions.cpp:840-852, which is only right for a symmetric matrix).
"""
import collections
import ctypes as C
import time

import numpy as np
import scipy.sparse as sp
import torch

from . import binding as _b

__all__ = ["clear_cache"]

_VP = C.c_void_p


def _require_gpu(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("sw_gcn: operands must live on the GPU (a ROCm 'cuda' tensor); "
                               "this build has no CPU executor")


def _stream():
    return _VP(torch.cuda.current_stream().cuda_stream)


class _Dense:
    """A torch tensor's memory seen as a tf_dense for the duration of one call."""

    def __init__(self, t):
        assert t.dtype == torch.float32 and t.is_contiguous() and t.dim() == 2
        self.t = t
        self.h = _VP()
        _b._check(_b.lib().tf_dense_wrap_device(t.shape[0], t.shape[1], _VP(t.data_ptr()), C.byref(self.h)))

    def __enter__(self):
        return self.h

    def __exit__(self, *exc):
        _b.lib().tf_dense_free(self.h)
        self.h = None


class _Adjacency:
    """Everything that is built once per adjacency matrix: the host copy of its pattern (the
    inspector runs on the host), the wrapped device CSR, schedules per (K, N), its transpose."""

    def __init__(self, adj):
        if adj.layout != torch.sparse_csr:
            raise RuntimeError("sw_gcn: Adj must be a sparse CSR tensor")
        crow, col, val = adj.crow_indices(), adj.col_indices(), adj.values()
        if crow.dtype != torch.int32 or col.dtype != torch.int32 or val.dtype != torch.float32:
            raise RuntimeError("sw_gcn: Adj needs int32 indices and float32 values, as in the reference")
        self.keep = (crow, col, val)  # the wrapped pointers stay valid while this object lives
        self.shape = tuple(adj.shape)
        self.device = adj.device
        self.Ap = np.ascontiguousarray(crow.cpu().numpy())
        self.Ai = np.ascontiguousarray(col.cpu().numpy())
        self.host = _b.CsrMatrix(self.shape[0], self.shape[1], self.Ap, self.Ai,
                                 np.zeros(max(1, len(self.Ai)), np.float32)[:len(self.Ai)])
        self.h = None
        self.schedules = {}
        self._t = None
        if adj.is_cuda:
            h = _VP()
            _b._check(_b.lib().tf_csr_wrap_device(self.shape[0], self.shape[1], int(self.Ap[-1]), _VP(crow.data_ptr()),
                                                 _VP(col.data_ptr()), _VP(val.data_ptr()), C.byref(h)))
            self.h = h
            # the device arrays were copied from the same tensors as the host pattern: let the executors
            # check schedules against it
            _b._check(_b.lib().tf_csr_set_pattern_hash(h, _b.pattern_hash(self.host)))

    def schedule(self, K, N):
        key = (K, N)
        if key not in self.schedules:
            self.schedules[key] = _b.inspector(self.host, 1, op=_b.OP_GEMM_SPMM, N=N, K=K)
        return self.schedules[key]

    def transpose(self):
        """The adjacency's transpose as another cached adjacency (itself when symmetric)."""
        if self._t is None:
            crow, col, val = self.keep
            m = sp.csr_matrix((val.cpu().numpy(), self.Ai, self.Ap), shape=self.shape)
            mt = m.T.tocsr()
            mt.sort_indices()
            ms = m.copy()
            ms.sort_indices()
            if mt.shape == ms.shape and np.array_equal(mt.indptr, ms.indptr) and np.array_equal(mt.indices, ms.indices) \
                    and np.array_equal(mt.data, ms.data):
                self._t = self
            else:
                t = torch.sparse_csr_tensor(torch.from_numpy(mt.indptr.astype(np.int32)), torch.from_numpy(mt.indices.astype(np.int32)),
                                            torch.from_numpy(mt.data.astype(np.float32)), size=mt.shape).to(self.device)
                self._t = _Adjacency(t)
        return self._t

    def __del__(self):
        if getattr(self, "h", None):
            _b.lib().tf_csr_free(self.h)
            self.h = None


_cache = collections.OrderedDict()
_CACHE_SIZE = 32


def _ctx(adj):
    crow, col, val = adj.crow_indices(), adj.col_indices(), adj.values()
    # the version counters change with every in-place update of the tensors: a cached host pattern,
    # schedule or transpose is never used for values or indices that were changed afterwards
    key = (crow.data_ptr(), col.data_ptr(), val.data_ptr(), tuple(adj.shape), int(val.numel()), str(adj.device),
           crow._version, col._version, val._version)
    c = _cache.get(key)
    if c is None:
        c = _Adjacency(adj)
        _cache[key] = c
        while len(_cache) > _CACHE_SIZE:
            _cache.popitem(last=False)
    else:
        _cache.move_to_end(key)
    return c


def clear_cache():
    """Drops the per-adjacency schedules and wrapped handles."""
    _cache.clear()


def _gemm_spmm(ctx, X, Wkn):
    """ctx.A @ (X @ Wkn) with X [M, K], Wkn [K, N], through tf_gemm_spmm."""
    _require_gpu(X, Wkn)
    M, K = X.shape
    N = Wkn.shape[1]
    if ctx.shape[1] != M or Wkn.shape[0] != K:
        raise RuntimeError(f"sw_gcn: shapes do not chain: Adj {ctx.shape}, Feature {tuple(X.shape)}, weight {tuple(Wkn.shape)}")
    X = X.to(torch.float32)
    Wkn = Wkn.to(torch.float32)
    X = X.contiguous()
    Wkn = Wkn.contiguous()
    out = torch.empty((ctx.shape[0], N), dtype=torch.float32, device=X.device)
    S = ctx.schedule(K, N)  # any K and N: the library pads K and cuts N into column panels itself
    with _Dense(X) as xb, _Dense(Wkn) as wc, _Dense(out) as db:
        _b._check(_b.lib().tf_gemm_spmm(ctx.h, xb, wc, db, S.h, 0, _stream()))
    return out


def _spmm(ctx, X):
    """ctx.A @ X through tf_spmm."""
    _require_gpu(X)
    X = X.to(torch.float32).contiguous()
    out = torch.empty((ctx.shape[0], X.shape[1]), dtype=torch.float32, device=X.device)
    with _Dense(X) as xb, _Dense(out) as ob:
        _b._check(_b.lib().tf_spmm(ctx.h, xb, ob, 0, _stream()))
    return out


class _FusedGeMMSpMM(torch.autograd.Function):
    """FusedGeMMSpMM / FusedGeMMSpMMROAdj (binding-project/src/Functions.cpp:1248-1268, 1192-1246):
    forward Adj @ (Feature @ Weight^T) with Weight [out, in]; backward for Feature and Weight."""

    @staticmethod
    def forward(fctx, adj, feature, weight):
        ctx = _ctx(adj)
        fctx.adj_ctx = ctx
        fctx.save_for_backward(feature, weight)
        return _gemm_spmm(ctx, feature, weight.t())

    @staticmethod
    def backward(fctx, grad_out):
        feature, weight = fctx.saved_tensors
        at = fctx.adj_ctx.transpose()
        grad_out = grad_out.contiguous()
        grad_feature = grad_weight = None
        if fctx.needs_input_grad[1]:
            grad_feature = _gemm_spmm(at, grad_out, weight)      # A^T (G W)
        if fctx.needs_input_grad[2]:
            grad_weight = torch.mm(_spmm(at, grad_out).t(), feature)  # (A^T G)^T X
        return None, grad_feature, grad_weight


def _schedule_tensors(ctx, K, N):
    v = ctx.schedule(K, N).view()
    P = int(v["ptr1_"][2])
    mix = np.empty(2 * P + 2, np.int32)
    mix[0:2 * P:2] = v["ptr2_"][:P]
    mix[1:2 * P:2] = v["ker_begin_"][0::2][:P]
    mix[2 * P] = v["ptr2_"][P]
    mix[2 * P + 1] = v["ptr2_"][P]
    return [torch.from_numpy(v["ptr1_"].astype(np.int32)), torch.from_numpy(mix), torch.from_numpy(v["id_"].astype(np.int32))]


# ---- operator implementations (names and argument orders of main.cpp:5-27) ----------------------

def inspect(Adj, MTileSize):
    del MTileSize
    return _schedule_tensors(_ctx(Adj), 64, 64)


def inspect_vt_ro(Adj, InDim, OutDim, CacheSize, NumThreads):
    del CacheSize, NumThreads
    return _schedule_tensors(_ctx(Adj), int(InDim), int(OutDim))


def executeFusedGeMMSpMM(Adj, Weight, Feature, LevelPtr, MixPtr, Partition, NumThreads):
    """Weight is [in, out] here, not transposed (main.cpp:76-103); returns (out, seconds)."""
    del LevelPtr, MixPtr, Partition, NumThreads
    _require_gpu(Adj, Weight, Feature)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = _gemm_spmm(_ctx(Adj), Feature, Weight)
    torch.cuda.synchronize()
    return [out, torch.tensor(time.perf_counter() - t0, dtype=torch.float32)]


def fusedGeMMSpMM(Adj, Feature, Weight, Schedule, NumThreads):
    del Schedule, NumThreads
    _require_gpu(Adj, Feature, Weight)
    return _FusedGeMMSpMM.apply(Adj, Feature, Weight)


def fusedGeMMSpMM_vt_ro(Adj, Feature, Weight, Schedule, NumThreads, MaxTileSize):
    del MaxTileSize
    return fusedGeMMSpMM(Adj, Feature, Weight, Schedule, NumThreads)


def geMMSpMM_f_bw(Adj, Feature, Weight, Schedule, NumThreads):
    return fusedGeMMSpMM(Adj, Feature, Weight, Schedule, NumThreads)


def cachedSpMMGeMM(AF, Weight, NumThreads):
    """ForwardCachingAF: (Adj @ Feature), computed once by the caller, times Weight^T."""
    del NumThreads
    return torch.mm(AF, Weight.t())


class _Unfused(torch.autograd.Function):
    """UnFusedGeMMSpMM: the two products as separate launches, the intermediate in HBM."""

    @staticmethod
    def forward(fctx, adj, feature, weight):
        _require_gpu(adj, feature, weight)
        ctx = _ctx(adj)
        fctx.adj_ctx = ctx
        fctx.save_for_backward(feature, weight)
        return _spmm(ctx, torch.mm(feature, weight.t()))

    @staticmethod
    def backward(fctx, grad_out):
        feature, weight = fctx.saved_tensors
        ag = _spmm(fctx.adj_ctx.transpose(), grad_out.contiguous())
        gf = torch.mm(ag, weight) if fctx.needs_input_grad[1] else None
        gw = torch.mm(ag.t(), feature) if fctx.needs_input_grad[2] else None
        return None, gf, gw


def unfused_gcn_forward(Adj, Feature, Weight, NumThreads):
    del NumThreads
    return _Unfused.apply(Adj, Feature, Weight)


def _two_layers(ctx, X, W1kn, W2kn, relu):
    """ctx.A @ (act(ctx.A @ (X @ W1kn)) @ W2kn) through tf_gcn_two_layers; the hidden layer never leaves the device."""
    _require_gpu(X, W1kn, W2kn)
    M, K = X.shape
    H, N = W1kn.shape[1], W2kn.shape[1]
    if ctx.shape[0] != ctx.shape[1] or ctx.shape[1] != M or W1kn.shape[0] != K or W2kn.shape[0] != H:
        raise RuntimeError(f"sw_gcn: shapes do not chain: Adj {ctx.shape}, Feature {tuple(X.shape)}, weights {tuple(W1kn.shape)}, {tuple(W2kn.shape)}")
    X = X.to(torch.float32).contiguous()
    W1 = W1kn.to(torch.float32).contiguous()
    W2 = W2kn.to(torch.float32).contiguous()
    out = torch.empty((M, N), dtype=torch.float32, device=X.device)
    s1, s2 = ctx.schedule(K, H), ctx.schedule(H, N)  # any widths: the library cuts column panels itself
    with _Dense(X) as xb, _Dense(W1) as w1, _Dense(W2) as w2, _Dense(out) as ob:
        _b._check(_b.lib().tf_gcn_two_layers(ctx.h, xb, w1, w2, ob, s1.h, s2.h, None, _b.RELU if relu else 0, _stream()))
    return out


def fusedGCN(Adj, Feature, Weight1, Weight2, NumThreads):
    """Two layers with a ReLU between, Adj @ (relu(Adj @ (Feature @ Weight1^T)) @ Weight2^T), weights [out, in]:
    the forward of the reference's end-to-end model (gcn-e2e-training/FusedGCNModule.py:14-18) and the
    composition its unregistered fusedGCN (binding-project/src/Functions.cpp:228-290) stands for.  When a
    gradient is wanted the two layers run as two fusedGeMMSpMM calls, whose backward passes exist."""
    del NumThreads
    _require_gpu(Adj, Feature, Weight1, Weight2)
    if torch.is_grad_enabled() and (Feature.requires_grad or Weight1.requires_grad or Weight2.requires_grad):
        return _FusedGeMMSpMM.apply(Adj, _FusedGeMMSpMM.apply(Adj, Feature, Weight1).relu(), Weight2)
    return _two_layers(_ctx(Adj), Feature, Weight1.t(), Weight2.t(), True)


SCHEMAS = {
    "inspect": "(Tensor Adj, int MTileSize) -> Tensor[]",
    "inspect_vt_ro": "(Tensor Adj, int InDim, int OutDim, int CacheSize, int NumThreads) -> Tensor[]",
    "executeFusedGeMMSpMM": "(Tensor Adj, Tensor Weight, Tensor Feature, Tensor LevelPtr, Tensor MixPtr, Tensor Partition, int NumThreads) -> Tensor[]",
    "fusedGeMMSpMM": "(Tensor Adj, Tensor Feature, Tensor Weight, Tensor[] Schedule, int NumThreads) -> Tensor",
    "fusedGeMMSpMM_vt_ro": "(Tensor Adj, Tensor Feature, Tensor Weight, Tensor[] Schedule, int NumThreads, int MaxTileSize) -> Tensor",
    "geMMSpMM_f_bw": "(Tensor Adj, Tensor Feature, Tensor Weight, Tensor[] Schedule, int NumThreads) -> Tensor",
    "cachedSpMMGeMM": "(Tensor AF, Tensor Weight, int NumThreads) -> Tensor",
    "unfused_gcn_forward": "(Tensor Adj, Tensor Feature, Tensor Weight, int NumThreads) -> Tensor",
    "fusedGCN": "(Tensor Adj, Tensor Feature, Tensor Weight1, Tensor Weight2, int NumThreads) -> Tensor",
}

_library = torch.library.Library("sw_gcn", "DEF")
for _name, _schema in SCHEMAS.items():
    _library.define(_name + _schema)
    _library.impl(_name, globals()[_name], "CompositeImplicitAutograd")
