"""The sw_gcn torch operators (the reference's binding-project/main.cpp:133-142 surface) over
libtilefusion_hip.  CPU tests: registration, schemas, the schedule tensors' layout, and that no
executor runs without a GPU.  GPU tests: forward and backward against dense torch fp64 and the
CPU oracle, to max|got - want| / max|want| <= 1e-4 (fp32 MFMA GEMM, sums in another order)."""
import importlib

import numpy as np
import pytest
import scipy.sparse as sp

torch = pytest.importorskip("torch")
ops_mod = importlib.import_module("tile-fusion_amd.torch_ops")
TOL = 1e-4


def csr_tensor(A, device="cpu"):
    A = A.tocsr()
    return torch.sparse_csr_tensor(torch.tensor(A.indptr, dtype=torch.int32), torch.tensor(A.indices, dtype=torch.int32),
                                   torch.tensor(A.data, dtype=torch.float32), size=A.shape).to(device)


def rel_err(got, want):
    got = got.detach().cpu().double().numpy()
    want = np.asarray(want, dtype=np.float64)
    return np.abs(got - want).max() / max(np.abs(want).max(), 1e-30)


def test_operators_are_registered_with_the_reference_signatures():
    for name, schema in ops_mod.SCHEMAS.items():
        op = getattr(torch.ops.sw_gcn, name)
        s = str(op.default._schema)
        assert s.startswith(f"sw_gcn::{name}(") and s.endswith(schema.split("->")[1].strip())
    args = [a.name for a in torch.ops.sw_gcn.fusedGeMMSpMM_vt_ro.default._schema.arguments]
    assert args == ["Adj", "Feature", "Weight", "Schedule", "NumThreads", "MaxTileSize"]
    args = [a.name for a in torch.ops.sw_gcn.executeFusedGeMMSpMM.default._schema.arguments]
    assert args == ["Adj", "Weight", "Feature", "LevelPtr", "MixPtr", "Partition", "NumThreads"]


def test_load_library_like_the_reference(tmp_path):
    """torch.ops.load_library("…/libsw_gcn.so"), the line the reference's Python layers start with
    (binding-project/gcn-e2e-training/FusedGCNLayer.py:3), in a fresh interpreter and from another directory:
    loading the library registers torch.ops.sw_gcn.* (it imports torch_ops.py), an inspector runs on CPU tensors."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = os.path.join(root, "tile-fusion_amd", "lib", "libsw_gcn.so")
    if not os.path.exists(lib):
        pytest.skip("libsw_gcn.so is not built")
    code = f"""
import torch
torch.ops.load_library({lib!r})
names = ["inspect", "inspect_vt_ro", "executeFusedGeMMSpMM", "fusedGeMMSpMM", "fusedGeMMSpMM_vt_ro", "geMMSpMM_f_bw",
         "cachedSpMMGeMM", "unfused_gcn_forward"]
assert all(hasattr(torch.ops.sw_gcn, n) for n in names)
crow = torch.arange(0, 9, dtype=torch.int32); col = torch.arange(0, 8, dtype=torch.int32)
adj = torch.sparse_csr_tensor(crow, col, torch.ones(8), size=(8, 8))
sched = torch.ops.sw_gcn.inspect_vt_ro(adj, 32, 32, 500000, 1)
assert len(sched) == 3
print("ok")
"""
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=600, cwd=str(tmp_path))
    assert r.returncode == 0 and "ok" in r.stdout, (r.stdout[-500:], r.stderr[-2000:])


def test_inspect_returns_the_binding_layout(tf):
    A = tf.workloads.banded_random(3000, 32, 16, seed=9)
    adj = csr_tensor(A)
    level, mix, part = torch.ops.sw_gcn.inspect_vt_ro(adj, 64, 64, 500000, 8)
    level, mix, part = level.numpy(), mix.numpy(), part.numpy()
    P0, P = level[1], level[2]
    assert level[0] == 0 and 0 < P0 <= P and len(mix) == 2 * P + 2 and len(part) == 2 * 3000
    assert np.all(np.diff(mix[:2 * P + 1]) >= 0) and mix[2 * P] == len(part)
    first = np.concatenate([part[mix[2 * p]:mix[2 * p + 1]] for p in range(P)])
    second = np.concatenate([part[mix[2 * p + 1]:mix[2 * p + 2]] for p in range(P)])
    assert np.array_equal(np.sort(first), np.arange(3000)) and np.array_equal(np.sort(second), np.arange(3000))
    for p in range(P0, P):  # remainder partitions hold second-op rows only
        assert mix[2 * p] == mix[2 * p + 1]
    level2, _, _ = torch.ops.sw_gcn.inspect(adj, 64)
    assert level2.shape == (3,)


def test_executors_refuse_cpu_tensors(tf):
    A = tf.workloads.laplacian_2d(8)
    adj = csr_tensor(A)
    sched = torch.ops.sw_gcn.inspect(adj, 16)
    with pytest.raises(RuntimeError, match="GPU"):
        torch.ops.sw_gcn.fusedGeMMSpMM(adj, torch.rand(64, 32), torch.rand(8, 32), sched, 1)
    with pytest.raises(RuntimeError, match="GPU"):
        torch.ops.sw_gcn.unfused_gcn_forward(adj, torch.rand(64, 32), torch.rand(8, 32), 1)
    bad = torch.sparse_csr_tensor(torch.tensor(A.indptr, dtype=torch.int64), torch.tensor(A.indices, dtype=torch.int64), torch.tensor(A.data, dtype=torch.float32))
    with pytest.raises(RuntimeError, match="int32"):
        torch.ops.sw_gcn.inspect(bad, 16)


@pytest.mark.gpu
@pytest.mark.parametrize("in_dim,out_dim", [(32, 5), (64, 64), (30, 7), (128, 128), (16, 300)])
def test_forward_matches_dense_reference(gpu, tf, orc, in_dim, out_dim):
    print(f"sw_gcn forward in={in_dim} out={out_dim}", flush=True)
    A = tf.workloads.erdos_renyi_gcn(3000, 8.0, seed=21)
    adj = csr_tensor(A, "cuda")
    g = torch.Generator().manual_seed(in_dim * 1000 + out_dim)
    x = torch.rand(3000, in_dim, generator=g)
    w = torch.rand(out_dim, in_dim, generator=g) - 0.5
    want = A.astype(np.float64) @ (x.double().numpy() @ w.double().numpy().T)
    sched = torch.ops.sw_gcn.inspect_vt_ro(adj, in_dim, out_dim, 500000, 8)
    out = torch.ops.sw_gcn.fusedGeMMSpMM_vt_ro(adj, x.cuda(), w.cuda(), sched, 8, 0)
    assert out.is_cuda and tuple(out.shape) == (3000, out_dim) and rel_err(out, want) <= TOL
    assert rel_err(torch.ops.sw_gcn.fusedGeMMSpMM(adj, x.cuda(), w.cuda(), sched, 8), want) <= TOL
    assert rel_err(torch.ops.sw_gcn.unfused_gcn_forward(adj, x.cuda(), w.cuda(), 8), want) <= TOL
    res = torch.ops.sw_gcn.executeFusedGeMMSpMM(adj, w.t().contiguous().cuda(), x.cuda(), sched[0], sched[1], sched[2], 8)
    assert rel_err(res[0], want) <= TOL and float(res[1]) > 0
    if in_dim % 8 == 0 and out_dim % 32 == 0 and out_dim <= 256:  # the reference's own CPU executor, restated
        o, _ = orc.gemm_spmm(A, x.numpy(), np.ascontiguousarray(w.numpy().T), orc.unfused_schedule(3000), nthreads=8)
        assert rel_err(out, o) <= TOL


@pytest.mark.gpu
@pytest.mark.parametrize("symmetric", [True, False])
def test_backward_matches_dense_autograd(gpu, tf, symmetric):
    print(f"sw_gcn backward symmetric={symmetric}", flush=True)
    n, in_dim, out_dim = 2000, 48, 24
    A = tf.workloads.erdos_renyi_gcn(n, 6.0, seed=22)
    if not symmetric:
        A = sp.triu(A, k=-3).tocsr() + sp.random(n, n, density=2.0 / n, random_state=3, format="csr", dtype=np.float32)
        A = A.tocsr().astype(np.float32)
    adj = csr_tensor(A, "cuda")
    g = torch.Generator().manual_seed(5)
    x0 = torch.rand(n, in_dim, generator=g)
    w0 = torch.rand(out_dim, in_dim, generator=g) - 0.5
    go = torch.rand(n, out_dim, generator=g) - 0.5
    xd = x0.double().requires_grad_()
    wd = w0.double().requires_grad_()
    Ad = torch.tensor(A.toarray(), dtype=torch.float64)
    (Ad @ (xd @ wd.t())).backward(go.double())
    for fn in (lambda a, x, w, s: torch.ops.sw_gcn.fusedGeMMSpMM_vt_ro(a, x, w, s, 8, 0),
               lambda a, x, w, s: torch.ops.sw_gcn.geMMSpMM_f_bw(a, x, w, s, 8),
               lambda a, x, w, s: torch.ops.sw_gcn.unfused_gcn_forward(a, x, w, 8)):
        x = x0.cuda().requires_grad_()
        w = w0.cuda().requires_grad_()
        sched = torch.ops.sw_gcn.inspect_vt_ro(adj, in_dim, out_dim, 500000, 8)
        fn(adj, x, w, sched).backward(go.cuda())
        assert rel_err(x.grad, xd.grad.numpy()) <= TOL and rel_err(w.grad, wd.grad.numpy()) <= TOL


@pytest.mark.gpu
def test_layer_written_like_the_reference(gpu, tf):
    """A module shaped like FusedGCNLayer (gcn-e2e-training/FusedGCNLayer.py:6-45) trains."""
    print("sw_gcn layer", flush=True)
    n = 1500
    A = tf.workloads.erdos_renyi_gcn(n, 6.0, seed=23)
    adj = csr_tensor(A, "cuda")

    class Layer(torch.nn.Module):
        def __init__(self, feat_dim, embed_dim):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.empty(embed_dim, feat_dim))
            torch.nn.init.xavier_uniform_(self.weight)
            self.schedule = torch.ops.sw_gcn.inspect_vt_ro(adj, feat_dim, embed_dim, 500000, 8)
            level_ptr, mix_ptr = self.schedule[0], self.schedule[1]
            self.max_tile_size = max(int(mix_ptr[2 * t + 2] - mix_ptr[2 * t]) for t in range(int(level_ptr[0]), int(level_ptr[1])))

        def forward(self, x):
            return torch.ops.sw_gcn.fusedGeMMSpMM_vt_ro(adj, x, self.weight, self.schedule, 8, self.max_tile_size)

    torch.manual_seed(0)
    net = torch.nn.Sequential(Layer(32, 64), torch.nn.ReLU(), Layer(64, 4)).cuda()
    x = torch.rand(n, 32, device="cuda")
    y = torch.randint(0, 4, (n,), device="cuda")
    opt = torch.optim.Adam(net.parameters(), lr=0.05)
    losses = []
    for _ in range(30):
        opt.zero_grad()
        loss = torch.nn.functional.cross_entropy(net(x), y)
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert losses[-1] < losses[0]


@pytest.mark.gpu
def test_two_layer_forward_op(gpu, tf):
    """sw_gcn.fusedGCN: both layers in one call with the hidden layer kept on the device, against
    float64; and with gradients wanted, against dense autograd."""
    print("sw_gcn fusedGCN", flush=True)
    n = 3000
    A = tf.workloads.erdos_renyi_gcn(n, 8.0, seed=29)
    adj = csr_tensor(A, "cuda")
    g = torch.Generator().manual_seed(7)
    for in_dim, hid, out_dim in ((64, 64, 32), (50, 40, 7), (128, 128, 128)):
        x0 = torch.rand(n, in_dim, generator=g)
        w1 = torch.rand(hid, in_dim, generator=g) - 0.5
        w2 = torch.rand(out_dim, hid, generator=g) - 0.5
        Ad = A.astype(np.float64)
        want = Ad @ (np.maximum(Ad @ (x0.double().numpy() @ w1.double().numpy().T), 0.0) @ w2.double().numpy().T)
        with torch.no_grad():
            got = torch.ops.sw_gcn.fusedGCN(adj, x0.cuda(), w1.cuda(), w2.cuda(), 8)
        assert got.shape == (n, out_dim) and rel_err(got, want) <= TOL, (in_dim, hid, out_dim)
    xd, w1d, w2d = x0.double().requires_grad_(), w1.double().requires_grad_(), w2.double().requires_grad_()
    Adt = torch.tensor(A.toarray(), dtype=torch.float64)
    go = torch.rand(n, out_dim, generator=g) - 0.5
    (Adt @ ((Adt @ (xd @ w1d.t())).relu() @ w2d.t())).backward(go.double())
    x, a1, a2 = x0.cuda().requires_grad_(), w1.cuda().requires_grad_(), w2.cuda().requires_grad_()
    torch.ops.sw_gcn.fusedGCN(adj, x, a1, a2, 8).backward(go.cuda())
    assert rel_err(x.grad, xd.grad.numpy()) <= TOL and rel_err(a1.grad, w1d.grad.numpy()) <= TOL and rel_err(a2.grad, w2d.grad.numpy()) <= TOL
