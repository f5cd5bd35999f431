#!/usr/bin/env python3
"""Benchmark of the fused executors on one MI355X.

One "step" is one pass of the hot path, D = A*(B*C), over one synthetic workload whose
operands are already resident in HBM.  With no flags the timed line is the largest
single-GPU configuration, the power-law GeMM-SpMM (R-MAT, 2^21 nodes, K = N = 128), and the
other four configurations are measured in the same process and reported under
"per_config".  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config {1..6}] [--only] [--unfused]
"""
import os

# the CPU leg follows the reference's protocol: threads pinned close together, no dynamic teams
# (must be in the environment before an OpenMP runtime is loaded)
os.environ.setdefault("OMP_PROC_BIND", "close")
os.environ.setdefault("OMP_DYNAMIC", "FALSE")

import argparse  # noqa: E402
import gc  # noqa: E402
import importlib  # noqa: E402
import json  # noqa: E402
import sys  # noqa: E402
import time  # noqa: E402

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

import numpy as np  # noqa: E402

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
MFMA_FP32_PEAK_TF = 157.3  # MI355X dense fp32 MFMA, published
LLC_BYTES = 256 << 20      # Infinity Cache
L2_GATHER_TBS = 19.7       # the row kernel gathering 512-byte rows that every XCD finds in its own L2 (profiles/calibration_gather.md)
METRIC = "fused GeMM-SpMM / SpMM-SpMM GFLOP/s and % HBM roofline, 1 MI355X vs CPU"
HEADLINE = 4               # largest single-GPU configuration, the power-law target


def _usable_cores():
    have = os.cpu_count() or 1
    try:
        have = min(have, len(os.sched_getaffinity(0)))
    except (AttributeError, OSError):
        pass
    return have


# taken before any OpenMP region runs: with OMP_PROC_BIND the runtime pins the calling thread to one
# core, after which the affinity mask no longer shows what the process may use
_USABLE_CORES = _usable_cores()


def cpu_threads():
    """Threads of the CPU leg: the cores this process may use.  The GPU boxes give a one-GPU job a
    share of the host and export it as OMP_NUM_THREADS; without that, every core the OS shows."""
    have = _USABLE_CORES
    env = os.environ.get("OMP_NUM_THREADS", "")
    limit = int(env.split(",")[0]) if env.split(",")[0].strip().isdigit() else 0
    return (min(have, limit) if limit > 0 else have), have, limit


def cpu_baseline(cfg, budget_s=40.0):
    """The reference's CPU executors on this box's host cores, on the same operands, by the
    reference's own protocol (scripts/run_exp.sh:133-158, scripts/plot.py:26-34): fused executor
    over variable-tile schedules for its six cache budgets and over fixed tiles of 16..2048
    rows, and the unfused pair of products.  Two passes, so that the whole sweep fits a bounded
    time: one trial of every variant, then seven trials (median) of the best fused variant and of
    the unfused pair -- what the reference's plots keep.  SpMM-SpMM runs the reference's own AVX2
    translation units (oracle/_ref) where they were built; GeMM-SpMM runs the C restatement, whose
    tile GEMM is a register-blocked AVX-512 micro-kernel where the host has AVX-512 (the class of
    kernel the reference gets from MKL's cblas_sgemm, which is not shipped here); its rate on
    this workload's GEMM alone is reported as gemm_gflops.  The CPU leg computes every row of the
    intermediate, as the reference does (it has no rule for rows nobody reads)."""
    import oracle_lib as O
    threads, have, limit = cpu_threads()
    threads = max(1, min(threads, O.max_threads()))
    A, N = cfg["A"], cfg["N"]
    flops = importlib.import_module("tile-fusion_amd").workloads.flops(cfg)
    gemm = cfg["op"] == "gemm_spmm"
    use_ref = (not gemm) and O.ref() is not None and N % 32 == 0 and cfg["B"] is A
    variants = [("variable tiles", c) for c in (500000, 1000000, 100000, 1500000, 60000, 1280000)]
    variants += [("fixed tiles", ip) for ip in (512, 128, 2048, 32, 1024, 256, 64, 16)]
    variants.insert(2, ("unfused", 0))
    t_start = time.perf_counter()

    def make(kind, par):
        if kind == "unfused":
            return None
        if kind == "variable tiles":
            return O.inspect_vt_gemm_spmm(A, cfg["K"], N, par) if gemm else O.inspect_vt_both_wavefronts(A, N, par, threads)
        return O.inspect_fixed_tiles(A, par, threads)

    def run(kind, S):
        t0 = time.perf_counter()
        if kind == "unfused":
            if gemm:
                O.spmm(A, O.gemm(cfg["B"], cfg["C"], nthreads=threads), nthreads=threads)
            elif use_ref:
                O.ref_spmm(A, O.ref_spmm(cfg["B"], cfg["C"], threads), threads)
            else:
                O.spmm(A, O.spmm(cfg["B"], cfg["C"], nthreads=threads), nthreads=threads)
        elif gemm:
            O.gemm_spmm(A, cfg["B"], cfg["C"], S, nthreads=threads)
        elif use_ref and kind == "fixed tiles":
            O.spmm_spmm_separated(A, cfg["C"], S, nthreads=threads, impl="ref")
        else:
            O.spmm_spmm(A, cfg["B"], cfg["C"], S, nthreads=threads, impl="ref_vec32" if use_ref else "oracle")
        return time.perf_counter() - t0

    # pass 1: every variant once (the first call of all is a warm-up and not counted)
    run("unfused", None)
    first, skipped = [], []
    for kind, par in variants:
        if time.perf_counter() - t_start > 0.6 * budget_s and first:
            skipped.append(f"{kind} {par}: time budget")
            continue
        try:
            S = make(kind, par)
        except ValueError:
            # (variable tiles: the reference's first tile is (cache / 4 - K N) / (K + N) rows, Fusion_Inspector.h:1029-1031,
            # which is negative when the cache budget is smaller than the weights)
            skipped.append(f"{kind} {par}: the inspector has no schedule for it (cache budget below K x N weights)")
            continue
        first.append((run(kind, S), kind, par, S))
    if not first:
        return None
    # pass 2: seven trials of the best fused variant and of the unfused pair
    fused1 = [r for r in first if r[1] != "unfused"]
    finals = ([min(fused1, key=lambda r: r[0])] if fused1 else []) + [r for r in first if r[1] == "unfused"]
    results, trials = [], len(first)
    for t1, kind, par, S in finals:
        times = [t1]
        while len(times) < 7 and time.perf_counter() - t_start < budget_s:
            times.append(run(kind, S))
        trials += len(times) - 1
        results.append((float(np.median(times)), kind, par, len(times)))
    gemm_gflops = None
    if gemm:  # the GEMM alone, all rows, same threads: how close the stand-in for MKL is to the host's FMA rate
        X, W = cfg["B"], cfg["C"]
        rows = min(X.shape[0], 1 << 19)
        O.gemm(X[:rows], W, nthreads=threads)
        t0 = time.perf_counter()
        O.gemm(X[:rows], W, nthreads=threads)
        gemm_gflops = round(2.0 * rows * X.shape[1] * W.shape[1] / (time.perf_counter() - t0) / 1e9, 1)
    best = min(results)
    fused = [r for r in results if r[1] != "unfused"]
    unf = [r for r in results if r[1] == "unfused"]
    return {"value": round(flops / best[0] / 1e9, 2), "unit": "GFLOP/s", "cores": threads,
            "kind": "reference" if use_ref else "port",
            "sample": f"full workload ({cfg['name']}) incl. zeroing of D and the intermediate; one trial of {len(first)} of the {len(variants)} "
                      f"variants of the reference's sweep, then the median of {best[3]} trials of the best fused variant and of the unfused pair; "
                      f"{trials} trials in {time.perf_counter() - t_start:.1f} s",
            "ms": round(best[0] * 1e3, 3),
            "best_variant": f"{best[1]} {best[2]}" if best[1] != "unfused" else "unfused",
            "best_fused_variant": f"{fused[0][1]} {fused[0][2]}" if fused else None,
            "best_fused_ms": round(fused[0][0] * 1e3, 3) if fused else None,
            "unfused_ms": round(unf[0][0] * 1e3, 3) if unf else None,
            "sweep_first_trial_ms": {f"{k} {p}" if k != "unfused" else k: round(t * 1e3, 2) for t, k, p, _ in first},
            "sweep_skipped": skipped,
            "gemm_gflops": gemm_gflops, "gemm_simd": ("avx512" if O.simd() else "avx2") if gemm else None,
            "os_cpu_count": os.cpu_count(), "usable_cores": have, "omp_num_threads_env": limit or None,
            "omp_proc_bind": os.environ.get("OMP_PROC_BIND"), "omp_dynamic": os.environ.get("OMP_DYNAMIC"),
            "note": ("the reference's own AVX2 kernels compiled from its sources" if use_ref else
                     "C restatement of the reference executor; its tile GEMM (gemm_gflops on this host) stands in for MKL cblas_sgemm, "
                     "which is not available here.  It computes all rows of the intermediate as the reference does; the GPU "
                     "executor skips the rows nobody reads (roofline.executed), so value / cpu value compares two amounts of GEMM work")}


def calibrate(tf, rows=1 << 20, N=128, reps=5):
    """A plain copy of known size: Y = X, device to device (tf_dense_copy; the runtime's copy
    kernel), reads rows*N*4 bytes and writes as many, with no reuse.  Run under
    `rocprofv3 --pmc FETCH_SIZE` (then WRITE_SIZE): the ratio of the counter to these byte
    counts is the factor the counter has to be scaled by."""
    X = tf.DenseMatrix(rows, N)
    X.fill(1.0)
    Y = tf.DenseMatrix(rows, N)
    tf.device_synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        Y.copy_from(X)
    tf.device_synchronize()
    dt = (time.perf_counter() - t0) / reps
    print(json.dumps({"calibration_kernel": "device-to-device copy (tf_dense_copy)", "launches": reps,
                      "read_bytes_per_launch": rows * N * 4, "write_bytes_per_launch": rows * N * 4,
                      "copy_GBps_read_plus_write": round(2 * rows * N * 4 / dt / 1e9, 1)}))


def calibrate_issue(tf, iters=2000):
    """Do the fp32 MFMA path and the VALU of a SIMD work at the same time?  One workgroup of eight wavefronts per compute
    unit (two per SIMD); the four older and the four younger wavefronts each run MFMAs, FMAs or nothing (tf_calibrate_issue)."""
    NONE, MFMA, FMA, BF16 = 0, 1, 2, 3
    cus = tf.device_init(0)["compute_units"]
    cases = [("fp32 MFMA on all eight", MFMA, MFMA), ("fp32 FMA on all eight", FMA, FMA),
             ("fp32 MFMA on the older four, the others idle", MFMA, NONE), ("fp32 FMA on the younger four, the others idle", NONE, FMA),
             ("fp32 MFMA on the older four beside fp32 FMA on the younger four", MFMA, FMA),
             ("fp32 FMA on the older four beside fp32 MFMA on the younger four", FMA, MFMA),
             ("bf16 MFMA on the older four, the others idle", BF16, NONE),
             ("bf16 MFMA on the older four beside fp32 FMA on the younger four", BF16, FMA)]
    out = {"calibration_kernel": "issue_probe_kernel via tf_calibrate_issue", "compute_units": cus, "rounds": iters,
           "per_round": "32 v_mfma_f32_16x16x4_f32 (65,536 flop) | 256 v_fma_f32 (32,768 flop) | 32 v_mfma_f32_16x16x32_bf16 per wavefront",
           "cases": []}
    for name, lo, hi in cases:
        ms = tf.calibrate_issue(lo, hi, iters)
        flop = sum(4 * cus * iters * {NONE: 0, MFMA: 32 * 2048, FMA: 256 * 128, BF16: 32 * 16384}[r] for r in (lo, hi))
        out["cases"].append({"case": name, "ms": round(ms, 4), "TFLOPs": round(flop / ms * 1e-9, 1)})
    print(json.dumps(out))


def calibrate_gather(tf, rows=1 << 19, per_row=32, N=128, reps=5):
    """The rate at which the row kernel (spmm_rows_kernel through tf_spmm) gathers 4N-byte rows when they are
    found in L2, in the Infinity Cache, or nowhere: Y = A X with `per_row` random columns per row drawn from
    (a) a region of 4 MB per XCD -- the row kernel deals workgroup b, i.e. rows 8b .. 8b+7 at N = 128, to XCD b mod 8,
    and row i draws from region (i / 8) mod 8, so every XCD gathers from its own 4 MB;
    (b) one region of 16 MB shared by all XCDs; (c) 1 GB.  gathered bytes = nnz * 4N; the rows of Y written
    (rows * 4N, streaming stores) come on top and are 1/per_row of that."""
    import scipy.sparse as sp
    rng = np.random.default_rng(77)
    out = {"calibration_kernel": "spmm_rows_kernel via tf_spmm", "rows": rows, "entries_per_row": per_row, "N": N, "launches": reps,
           "gathered_bytes_per_launch": rows * per_row * 4 * N, "cases": []}
    row_bytes = 4 * N
    g = 256 // max(8, N // 4)  # rows per workgroup of the row kernel
    cases = [("own 4 MB per XCD", 8 * (4 << 20) // row_bytes, lambda i: ((i // g) % 8) * ((4 << 20) // row_bytes), (4 << 20) // row_bytes),
             ("one 16 MB for all XCDs", (16 << 20) // row_bytes, lambda i: 0 * i, (16 << 20) // row_bytes),
             ("1 GB", (1 << 30) // row_bytes, lambda i: 0 * i, (1 << 30) // row_bytes)]
    for name, x_rows, base, span in cases:
        i = np.repeat(np.arange(rows), per_row)
        cols = base(i) + rng.integers(0, span, size=rows * per_row)
        A = sp.csr_matrix((np.ones(rows * per_row, np.float32), cols.astype(np.int32), np.arange(0, rows * per_row + 1, per_row, dtype=np.int32)),
                          shape=(rows, x_rows))
        Ah = tf.CsrMatrix.from_scipy(A).to_device()
        X = tf.DenseMatrix(x_rows, N)
        X.fill(1.0)
        Y = tf.DenseMatrix(rows, N)
        st = tf.Stream()
        tf.spmm(Ah, X, Y, stream=st)
        st.synchronize()
        e0, e1 = tf.Event(), tf.Event()
        e0.record(st)
        for _ in range(reps):
            tf.spmm(Ah, X, Y, stream=st)
        e1.record(st)
        st.synchronize()
        ms = e0.elapsed_ms(e1) / reps
        out["cases"].append({"gathers_from": name, "ms": round(ms, 4), "gather_TBps": round(rows * per_row * row_bytes / ms / 1e9, 2)})
        del Ah, X, Y
        gc.collect()
    print(json.dumps(out))


def check_result(cfg, got, max_rows=1 << 17, W2=None):
    """max |got - want| / max |want| against float64, on every row or -- for the configurations with
    millions of rows -- on a fixed sample of rows that includes the longest ones.  W2: the second layer's
    weights, for a two-layer step (ReLU between the layers)."""
    A = cfg["A"]
    L = A.shape[0]
    t = cfg["B"].astype(np.float64) @ cfg["C"].astype(np.float64)
    if W2 is not None:
        t = np.maximum(A.astype(np.float64) @ t, 0.0) @ W2.astype(np.float64)
    if L <= max_rows:
        rows = None
        want = A.astype(np.float64) @ t
    else:
        rng = np.random.default_rng(1234)
        longest = np.argsort(np.diff(A.indptr))[-64:]
        rows = np.unique(np.concatenate([rng.choice(L, max_rows, replace=False), longest]))
        want = A[rows].astype(np.float64) @ t
        got = got[rows]
    err = float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))
    return err, (L if rows is None else int(rows.size))


def kernel_names(info, op_is_gemm, unfused):
    if unfused:
        return "gemm_rows_kernel + spmm_rows_kernel"
    if not op_is_gemm:
        return ("fused_spmm_spmm_march_kernel" if info["marched"] else
                "fused_spmm_spmm_window64_kernel" if info["wide_strips"] else
                "fused_spmm_spmm_window_kernel" if info["windowed"] else
                "fused_spmm_spmm_kernel" if info["n_fused_rows"] else "spmm_rows_kernel (twice)")
    if info["n_fused_rows"] == 0:
        return "gemm_rows_kernel + spmm_rows_kernel" + (" (+ long-row segments)" if info["n_long_rows"] else "")
    return ("fused_gemm_spmm_stream_kernel" if info["streamed"] else
            "fused_gemm_spmm_regw_kernel" if info["register_weights"] else "fused_gemm_spmm_kernel")


def run_config(tf, cfg, idx, steps, warmup, args):
    """Builds the schedule, times `steps` steps after `warmup`, checks the result."""
    w = tf.workloads
    A, N, K = cfg["A"], cfg["N"], cfg["K"]
    gemm = cfg["op"] == "gemm_spmm"
    op = tf.OP_GEMM_SPMM if gemm else tf.OP_SPMM_SPMM
    Ah = tf.CsrMatrix.from_scipy(A).to_device()
    t0 = time.perf_counter()
    inner = Ah if (not gemm and cfg["B"] is A and not args.no_window) else None
    S = tf.inspector(Ah, 1, op=op, N=N, K=K, lds_budget_bytes=args.lds, tile_rows=args.tile_rows,
                     max_redundancy=args.max_redundancy, inner=inner, strip_cols=args.strip, wide_strips=args.wide,
                     long_row_nnz=args.long_row, xcd_chunk_rows=args.xcd_chunk, long_row_partition=args.long_part,
                     march=args.march, reorder_adjacency=args.reorder_adj)
    inspect_s = time.perf_counter() - t0
    S.validate()
    info = S.info()
    Cd = tf.DenseMatrix.from_numpy(cfg["C"])
    D = tf.DenseMatrix(A.shape[0], N)
    second = bool(args.second_stream)
    if not gemm:
        Bh = Ah if cfg["B"] is A else tf.CsrMatrix.from_scipy(cfg["B"]).to_device()
        step = lambda st: tf.spmm_spmm(Ah, Bh, Cd, D, S, stream=st, second_stream=second)  # noqa: E731
    else:
        Bd = tf.DenseMatrix.from_numpy(cfg["B"])
        step = lambda st: tf.gemm_spmm(Ah, Bd, Cd, D, S, stream=st, second_stream=second)  # noqa: E731
        if args.unfused:  # the two products as separate launches, the intermediate through HBM
            T = tf.DenseMatrix(A.shape[1], N)
            step = lambda st: (tf.gemm(Bd, Cd, T, stream=st), tf.spmm(Ah, T, D, stream=st))  # noqa: E731
        if args.two_layers:  # D = A (relu(A (B C)) W2): tf_gcn_two_layers, one schedule for both layers (K = N)
            if K != N or A.shape[0] != A.shape[1]:
                sys.exit("bench.py --two-layers: needs a square matrix and K = N (e.g. --config 6)")
            W2 = w.uniform((N, N), 14)
            W2d = tf.DenseMatrix.from_numpy(W2)
            fuse = args.two_layers == "fuse"
            step = lambda st: tf.gcn_two_layers(Ah, Bd, Cd, W2d, D, S, S, relu=True, fuse=fuse, stream=st)  # noqa: E731

    st = tf.Stream()
    for _ in range(warmup):
        step(st)
    st.synchronize()
    tf.device_synchronize()
    e0, e1 = tf.Event(), tf.Event()
    t0 = time.perf_counter()
    e0.record(st)
    for _ in range(steps):
        step(st)
    e1.record(st)
    st.synchronize()
    tf.device_synchronize()
    wall = time.perf_counter() - t0
    dev_ms = e0.elapsed_ms(e1) / steps   # HIP events on the launch stream
    ms_per_step = wall * 1e3 / steps

    # one more step with events around every launch
    kernels = []
    if not args.unfused:
        S.set_profiling(True)
        step(st)
        kernels = [{"name": n, "ms": round(ms, 5)} for n, ms in S.profile()]
        S.set_profiling(False)

    err, rows_checked = (None, 0)
    if not args.no_check:
        err, rows_checked = check_result(cfg, D.to_numpy(), W2=W2 if (gemm and args.two_layers) else None)
        if not err <= 1e-4:
            print(f"bench.py: result check failed on {cfg['name']}, rel err {err:.3e}", file=sys.stderr)
            sys.exit(1)

    flops = w.flops(cfg)
    alg_bytes = w.algorithmic_bytes(cfg)
    gemm_flops = 2.0 * A.shape[1] * K * N if gemm else 0.0
    if gemm and args.two_layers:  # both layers; compulsory bytes: the hidden layer never leaves the chip, A is read once
        flops, gemm_flops = 2.0 * flops, 2.0 * gemm_flops
        alg_bytes += 4.0 * N * N
    t_hbm = alg_bytes / (HBM_PEAK_GBS * 1e9)
    t_mfma = gemm_flops / (MFMA_FP32_PEAK_TF * 1e12)
    bound = "mfma" if t_mfma > t_hbm else "hbm"
    dev_s = dev_ms * 1e-3
    operand_bytes = alg_bytes + (4.0 * A.shape[1] * N if info["n_writeback_rows"] else 0.0)
    # What was executed, beside the nominal work model: the GEMM of the intermediate rows the executor computes
    # (halo rows recomputed by tiles count, rows nobody reads do not), their rows of B instead of all of B; and the
    # bytes gathered through the caches by rows that did not fuse (4N per stored entry), which at the row kernel's
    # measured rate out of L2 (profiles/calibration_gather.md) is a third roof for steps that gather.
    computed = info["n_computed_rows"]
    exe_gemm_flops = 2.0 * computed * K * N if gemm else 0.0
    exe_bytes = alg_bytes - 4.0 * (A.shape[1] - computed) * K if gemm else alg_bytes
    gathered = 4.0 * N * (A.nnz - info["fused_nnz"])
    if not gemm and info["n_fused_rows"] == 0:
        gathered += 4.0 * N * cfg["B"].nnz
    t_exe = max(exe_bytes / (HBM_PEAK_GBS * 1e9), exe_gemm_flops / (MFMA_FP32_PEAK_TF * 1e12))
    t_gather = gathered / (L2_GATHER_TBS * 1e12)
    res = {
        "cfg": idx, "workload": cfg["name"], "op": cfg["op"], "rows": int(A.shape[0]), "nnz": int(A.nnz), "N": N, "K": K,
        "ms_per_step": round(ms_per_step, 5), "kernel_ms": round(dev_ms, 5),
        "gflops": round(flops / (ms_per_step * 1e-3) / 1e9, 2),
        "bound": bound, "frac": round(max(t_hbm, t_mfma) / dev_s, 4),
        "hbm_frac": round(t_hbm / dev_s, 4), "mfma_frac": round(t_mfma / dev_s, 4) if gemm else None,
        "algorithmic_bytes": int(alg_bytes), "gemm_flops": int(gemm_flops), "flops": int(flops),
        "executed": {"computed_intermediate_rows": int(computed), "gemm_flops": int(exe_gemm_flops), "bytes": int(exe_bytes),
                     "bound": "mfma" if exe_gemm_flops / (MFMA_FP32_PEAK_TF * 1e12) > exe_bytes / (HBM_PEAK_GBS * 1e9) else "hbm",
                     "frac": round(t_exe / dev_s, 4),
                     "mfma_TFLOPs": round(exe_gemm_flops / dev_s / 1e12, 2) if gemm else None},
        "gather": {"gathered_bytes": int(gathered), "l2_gather_TBps": L2_GATHER_TBS, "frac": round(t_gather / dev_s, 4)} if gathered else None,
        "working_set_vs_llc": round(operand_bytes / LLC_BYTES, 2),
        "rel_err_vs_f64": err, "rows_checked": rows_checked,
        "kernels": kernels, "kernel": ("fused_gcn2_kernel" if args.two_layers == "fuse" else "2 x " + kernel_names(info, gemm, False) + " + relu_kernel")
        if (gemm and args.two_layers) else kernel_names(info, gemm, args.unfused),
        "schedule": {"lds_bytes": info["lds_bytes"], "windowed": bool(info["windowed"]), "wide_strips": bool(info["wide_strips"]),
                     "streamed": bool(info["streamed"]), "marched": bool(info["marched"]), "tiles": info["n_tiles"], "fused_rows": info["n_fused_rows"],
                     "remainder_rows": info["n_remainder_rows"], "long_rows": info["n_long_rows"],
                     "long_row_hot_cols": info["long_row_hot_cols"],
                     "recomputed_rows": info["n_producer_rows"] - A.shape[1], "writeback_rows": info["n_writeback_rows"],
                     "inspector_s": round(inspect_s, 4)},
    }
    try:  # measured HBM traffic of the step's kernels, if a committed profile covers this schedule
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            t = json.load(f).get(f"cfg{idx}")
        if t and t["kernel"] == res["kernel"] and t["tiles"] == info["n_tiles"]:
            res["traffic"] = t["fetch_bytes"] + t["write_bytes"]
            res["traffic_source"] = t["source"]
    except (OSError, ValueError, KeyError):
        pass
    return res, (Ah, S)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=HEADLINE, choices=[1, 2, 3, 4, 5, 6, 7],
                    help="the configuration of the timed line (default: 4, the largest)")
    ap.add_argument("--only", action="store_true", help="skip the per_config table of the other configurations")
    ap.add_argument("--lds", type=int, default=0, help="LDS budget per tile in bytes (0 = library default)")
    ap.add_argument("--tile-rows", type=int, default=0)
    ap.add_argument("--max-redundancy", type=float, default=0.0)
    ap.add_argument("--strip", type=int, default=0, help="columns per strip of windowed tiles (32 or 64)")
    ap.add_argument("--no-window", action="store_true", help="do not build windowed tiles")
    ap.add_argument("--wide", type=int, default=0, choices=[-1, 0, 1],
                    help="windowed tiles: 1 = the 64-column, 1024-thread kernel, -1 = the lane-group kernel, 0 = library's choice")
    ap.add_argument("--xcd-chunk", type=int, default=0, help="rows per XCD turn of the row kernels (-1 contiguous)")
    ap.add_argument("--long-row", type=int, default=0, help="rows with more entries than this are chunked")
    ap.add_argument("--long-part", type=int, default=0, choices=[-1, 0, 1],
                    help="long rows: 1 = regrouped by the XCD partition of their columns, -1 = chunks of consecutive entries, 0 = library's choice")
    ap.add_argument("--march", type=int, default=0, choices=[-1, 0, 1], help="marching runs for stencils on 3D grids: -1 = never, 1 = must")
    ap.add_argument("--reorder-adj", type=int, default=0, choices=[-1, 0, 1],
                    help="remainder rows: -1 = read from A's arrays through the row list, 0/1 = stored in list order (reordered adjacency)")
    ap.add_argument("--second-stream", action="store_true", help="hot long-row segments on the executor's second stream, beside the GEMM (TF_SECOND_STREAM)")
    ap.add_argument("--matrix", default=None, help="run on a .mtx / .smtx file instead of a synthetic configuration "
                    "(square; symmetric files are expanded), with --op, --N and --K")
    ap.add_argument("--op", default="spmm_spmm", choices=["spmm_spmm", "gemm_spmm"])
    ap.add_argument("--N", type=int, default=64)
    ap.add_argument("--K", type=int, default=64)
    ap.add_argument("--scramble", action="store_true",
                    help="permute the rows and columns of the (square) matrix at random first")
    ap.add_argument("--rcm", action="store_true",
                    help="reorder the matrix with tf_reorder_rcm / tf_permute_csr before inspecting it (after --scramble)")
    ap.add_argument("--partition", type=int, default=0,
                    help="renumber the graph with tf_reorder_partition into this many parts first (hubs in front)")
    ap.add_argument("--unfused", action="store_true",
                    help="GeMM-SpMM as two launches (tf_gemm, tf_spmm) with the intermediate in HBM, for comparison")
    ap.add_argument("--two-layers", default=None, choices=["compose", "fuse"],
                    help="GeMM-SpMM with K = N on a square matrix (--config 6): two GCN layers per step through tf_gcn_two_layers, "
                         "as one executor call per layer or through the schedule's two-layer tiles (TF_FUSE_LAYERS)")
    ap.add_argument("--host-buffers", action="store_true",
                    help="also time the step as the README API runs it on un-pinned operands: upload A, B/C and D, "
                         "execute, download D (reported as host_buffer_ms_per_step; never part of value)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-check", action="store_true", help="skip the result check")
    ap.add_argument("--calibrate", action="store_true",
                    help="run a copy of known size instead (scales rocprofv3's FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--calibrate-issue", action="store_true",
                    help="time fp32 MFMA and fp32 VALU work of two wavefronts of a SIMD, alone and side by side")
    ap.add_argument("--calibrate-gather", action="store_true",
                    help="measure the row kernel's gather rate out of L2 / the Infinity Cache / HBM instead (the gather roof's rate)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported "
              "(more GPUs would each take a block of rows of A and D; no such path is built)", file=sys.stderr)
        sys.exit(2)

    tf = importlib.import_module("tile-fusion_amd")
    w = tf.workloads
    dev = tf.device_init(0)
    if args.calibrate:
        calibrate(tf)
        return
    if args.calibrate_issue:
        calibrate_issue(tf)
        return
    if args.calibrate_gather:
        calibrate_gather(tf)
        return
    custom = bool(args.matrix or args.scramble or args.rcm or args.partition or args.unfused or args.two_layers)
    if args.matrix:
        Af = tf.read_matrix(args.matrix)
        if Af.shape[0] != Af.shape[1]:
            sys.exit("bench.py --matrix: the matrix must be square")
        Mf = Af.shape[0]
        gemm = args.op == "gemm_spmm"
        cfg = dict(op=args.op, A=Af, B=w.uniform((Mf, args.K), 21) if gemm else Af, C=w.uniform((args.K if gemm else Mf, args.N), 22),
                   K=args.K if gemm else 0, N=args.N, name=f"file {os.path.basename(args.matrix)} {args.op} N={args.N}" + (f" K={args.K}" if gemm else ""))
    else:
        cfg = w.make_config(args.config)
    if args.two_layers:
        cfg["name"] += ", two layers with ReLU (tf_gcn_two_layers: " + ("two-layer tiles, hidden layer in LDS)" if args.two_layers == "fuse" else "one executor call per layer)")
    reorder_s = None
    if args.scramble or args.rcm or args.partition:  # same product on a renumbered graph: A' = A[p,:][:,p], dense row operands follow
        A0 = cfg["A"]
        if A0.shape[0] != A0.shape[1]:
            sys.exit("bench.py --scramble/--rcm/--partition: the matrix must be square")
        same_b = cfg["B"] is A0
        rows_follow = ["B"] if cfg["op"] == "gemm_spmm" else ["C"]
        if args.scramble:
            p = np.random.default_rng(5).permutation(A0.shape[0]).astype("int32")
            A0 = tf.permute_csr(A0, p)
            for k in rows_follow:
                cfg[k] = cfg[k][p]
            cfg["name"] += ", scrambled"
        if args.rcm:
            t0 = time.perf_counter()
            p = tf.reorder_rcm(A0)
            A0 = tf.permute_csr(A0, p)
            reorder_s = time.perf_counter() - t0
            for k in rows_follow:
                cfg[k] = cfg[k][p]
            cfg["name"] += ", RCM"
        if args.partition:
            t0 = time.perf_counter()
            p, _ = tf.reorder_partition(A0, args.partition)
            A0 = tf.permute_csr(A0, p)
            reorder_s = time.perf_counter() - t0
            for k in rows_follow:
                cfg[k] = cfg[k][p]
            cfg["name"] += f", partition ordering ({args.partition} parts, hubs in front)"
        cfg["A"] = A0
        if same_b:
            cfg["B"] = A0

    # steps for the small configurations: enough launches for a stable mean
    def steps_for(c):
        return args.steps if c["A"].shape[0] >= 1 << 20 else max(args.steps, 200)

    head_steps = args.steps  # the timed line runs exactly the steps asked for
    head, keep = run_config(tf, cfg, args.config, head_steps, args.warmup, args)
    A = cfg["A"]
    out = {
        "metric": METRIC, "value": head["gflops"], "unit": "GFLOP/s", "n_gpus": 1,
        "steps": head_steps,
        "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": cfg["name"], "op": cfg["op"], "rows": int(A.shape[0]), "nnz": int(A.nnz), "N": cfg["N"], "K": cfg["K"],
                   **head["schedule"], "kernels_per_step": len(head["kernels"]) or None,
                   "working_set_vs_llc": head["working_set_vs_llc"],
                   **({"reorder_s": round(reorder_s, 4)} if reorder_s is not None else {}),
                   "rel_err_vs_f64": head["rel_err_vs_f64"], "rows_checked": head["rows_checked"], "device": dev["arch"],
                   "xcd_round_robin_verified": dev["xcd_round_robin"]},
    }
    dev_s = head["kernel_ms"] * 1e-3
    hbm = {"achieved": round(head["algorithmic_bytes"] / dev_s / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": head["hbm_frac"]}
    if head["bound"] == "mfma":
        ach = head["gemm_flops"] / dev_s / 1e12
        roof = {"bound": "mfma", "achieved": round(ach, 2), "peak": MFMA_FP32_PEAK_TF, "unit": "TFLOP/s", "frac": round(ach / MFMA_FP32_PEAK_TF, 4),
                "hbm": hbm}
    else:
        roof = {"bound": "hbm", **hbm}
    roof.update({"traffic": head.get("traffic"), "algorithmic_bytes": head["algorithmic_bytes"], "gemm_flops": head["gemm_flops"],
                 "executed": head["executed"], "gather": head["gather"],
                 "kernel_ms": head["kernel_ms"], "kernel": head["kernel"], "kernels": head["kernels"],
                 "note": "a step is several launches: achieved = NOMINAL algorithmic work of the whole step (2 M K N for the GEMM, every row of B) / "
                         "HIP-event time of the step on the launch stream; `executed` = the same fraction on the work the executor does "
                         "(the GEMM only of intermediate rows some row of A reads, their rows of B); `gather` = bytes the unfused rows "
                         "gather through the caches / the row kernel's measured rate out of L2, as a fraction of the step: what a "
                         "formulation that gathers could reach at best; `kernels` = each launch timed by its own events in one extra "
                         "step (launches on the executor's second stream run beside the others, so the list can add up to more than kernel_ms)"})
    if "traffic_source" in head:
        roof["traffic_source"] = head["traffic_source"]
    out["roofline"] = roof

    if args.host_buffers:  # PCIe-inclusive: every operand crosses the bus each step
        N = cfg["N"]
        op = tf.OP_GEMM_SPMM if cfg["op"] == "gemm_spmm" else tf.OP_SPMM_SPMM
        S = keep[1]
        reps = 5
        t0 = time.perf_counter()
        for _ in range(reps):
            Ah2 = tf.CsrMatrix.from_scipy(A).to_device()
            Cd2 = tf.DenseMatrix.from_numpy(cfg["C"])
            D2 = tf.DenseMatrix(A.shape[0], N, np.zeros((A.shape[0], N), np.float32))
            if op == tf.OP_SPMM_SPMM:
                tf.spmm_spmm(Ah2, Ah2 if cfg["B"] is A else tf.CsrMatrix.from_scipy(cfg["B"]).to_device(), Cd2, D2, S, accumulate=True)
            else:
                tf.gemm_spmm(Ah2, tf.DenseMatrix.from_numpy(cfg["B"]), Cd2, D2, S, accumulate=True)
            D2.to_numpy()
        out["host_buffer_ms_per_step"] = round((time.perf_counter() - t0) * 1e3 / reps, 3)
    del keep
    gc.collect()

    if not custom and not args.only:  # the other configurations, same process, same protocol
        per = []
        for idx in (1, 2, 3, 4, 5):
            if idx == args.config:
                continue
            c = w.make_config(idx)
            r, keep = run_config(tf, c, idx, steps_for(c), args.warmup, args)
            r.pop("schedule")
            per.append(r)
            del c, keep
            gc.collect()
        out["per_config"] = per
    # last, because the OpenMP runtime pins this thread once its first region has run
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
