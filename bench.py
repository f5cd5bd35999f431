#!/usr/bin/env python3
"""Benchmark of the fused executors on one MI355X.

One "step" is one pass of the hot path, D = A*(B*C), over one synthetic workload whose
operands are already resident in HBM.  Default workload: the banded SpMM-SpMM
configuration (65,536 rows, bandwidth 32, N = 128).  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config {1..6}] [--unfused]
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

import numpy as np  # noqa: E402

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
MFMA_FP32_PEAK_TF = 157.3  # MI355X dense fp32 MFMA, published
METRIC = "fused GeMM-SpMM / SpMM-SpMM GFLOP/s and % HBM roofline, 1 MI355X vs CPU"


def cpu_baseline(cfg, budget_s=20.0):
    """The reference's CPU executor on this box's host cores, on the same operands.
    SpMM-SpMM: the reference's own AVX2 kernel compiled from its sources (oracle/_ref),
    over schedules from the restated variable-tile inspector; GeMM-SpMM: the C restatement
    (its GEMM is MKL in the reference).  Median of up to 7 trials per cache budget, best
    budget kept (the reference's protocol), bounded by `budget_s` seconds."""
    import oracle_lib as O
    threads = min(os.cpu_count() or 1, O.max_threads(), 16)
    A, N = cfg["A"], cfg["N"]
    flops = importlib.import_module("tile-fusion_amd").workloads.flops(cfg)
    best, best_cache, trials_done = None, None, 0
    t_start = time.perf_counter()
    use_ref = cfg["op"] == "spmm_spmm" and O.ref() is not None and N % 32 == 0
    for cache in (500000, 1000000, 100000, 1500000, 60000, 1280000):
        if time.perf_counter() - t_start > budget_s:
            break
        try:
            if cfg["op"] == "spmm_spmm":
                S = O.inspect_vt_both_wavefronts(A, N, cache, threads)
            else:
                S = O.inspect_vt_gemm_spmm(A, cfg["K"], N, cache)
        except ValueError:
            continue
        times = []
        for _ in range(7):
            t0 = time.perf_counter()
            if cfg["op"] == "spmm_spmm":
                O.spmm_spmm(A, cfg["B"], cfg["C"], S, nthreads=threads, impl="ref_vec32" if use_ref else "oracle")
            else:
                O.gemm_spmm(A, cfg["B"], cfg["C"], S, nthreads=threads)
            times.append(time.perf_counter() - t0)
            trials_done += 1
            if time.perf_counter() - t_start > budget_s and len(times) >= 3:
                break
        med = float(np.median(times))
        if best is None or med < best:
            best, best_cache = med, cache
    if best is None:
        return None
    return {"value": round(flops / best / 1e9, 2), "unit": "GFLOP/s", "cores": threads,
            "kind": "reference" if use_ref else "port",
            "sample": f"full workload incl. zeroing of D and the intermediate, median of <=7 trials per cache budget, "
                      f"best budget {best_cache} B, {trials_done} trials in {time.perf_counter() - t_start:.1f} s",
            "ms": round(best * 1e3, 3)}


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=2, choices=[1, 2, 3, 4, 5, 6])
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
    ap.add_argument("--matrix", default=None, help="run on a .mtx / .smtx file instead of a synthetic configuration "
                    "(square; symmetric files are expanded), with --op, --N and --K")
    ap.add_argument("--op", default="spmm_spmm", choices=["spmm_spmm", "gemm_spmm"])
    ap.add_argument("--N", type=int, default=64)
    ap.add_argument("--K", type=int, default=64)
    ap.add_argument("--scramble", action="store_true",
                    help="permute the rows and columns of the (square) matrix at random first")
    ap.add_argument("--rcm", action="store_true",
                    help="reorder the matrix with tf_reorder_rcm / tf_permute_csr before inspecting it (after --scramble)")
    ap.add_argument("--unfused", action="store_true",
                    help="GeMM-SpMM as two launches (tf_gemm, tf_spmm) with the intermediate in HBM, for comparison")
    ap.add_argument("--host-buffers", action="store_true",
                    help="also time the step as the README API runs it on un-pinned operands: upload A, B/C and D, "
                         "execute, download D (reported as host_buffer_ms_per_step; never part of value)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-check", action="store_true", help="skip the result check")
    ap.add_argument("--calibrate", action="store_true",
                    help="run a copy of known size instead (scales rocprofv3's FETCH_SIZE / WRITE_SIZE)")
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
    reorder_s = None
    if args.scramble or args.rcm:  # same product on a renumbered graph: A' = A[p,:][:,p], dense row operands follow
        A0 = cfg["A"]
        if A0.shape[0] != A0.shape[1]:
            sys.exit("bench.py --scramble/--rcm: the matrix must be square")
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
        cfg["A"] = A0
        if same_b:
            cfg["B"] = A0
    A, N, K = cfg["A"], cfg["N"], cfg["K"]
    op = tf.OP_GEMM_SPMM if cfg["op"] == "gemm_spmm" else tf.OP_SPMM_SPMM

    Ah = tf.CsrMatrix.from_scipy(A).to_device()
    t0 = time.perf_counter()
    inner = Ah if (op == tf.OP_SPMM_SPMM and cfg["B"] is A and not args.no_window) else None
    S = tf.inspector(Ah, 1, op=op, N=N, K=K, lds_budget_bytes=args.lds, tile_rows=args.tile_rows,
                     max_redundancy=args.max_redundancy, inner=inner, strip_cols=args.strip, wide_strips=args.wide,
                     long_row_nnz=args.long_row, xcd_chunk_rows=args.xcd_chunk, long_row_partition=args.long_part)
    inspect_s = time.perf_counter() - t0
    S.validate()
    info = S.info()
    Cd = tf.DenseMatrix.from_numpy(cfg["C"])
    D = tf.DenseMatrix(A.shape[0], N)
    if op == tf.OP_SPMM_SPMM:
        Bh = Ah if cfg["B"] is A else tf.CsrMatrix.from_scipy(cfg["B"]).to_device()
        step = lambda st: tf.spmm_spmm(Ah, Bh, Cd, D, S, stream=st)  # noqa: E731
    else:
        Bd = tf.DenseMatrix.from_numpy(cfg["B"])
        step = lambda st: tf.gemm_spmm(Ah, Bd, Cd, D, S, stream=st)  # noqa: E731
        if args.unfused:  # the two products as separate launches, the intermediate through HBM
            T = tf.DenseMatrix(A.shape[1], N)
            step = lambda st: (tf.gemm(Bd, Cd, T, stream=st), tf.spmm(Ah, T, D, stream=st))  # noqa: E731

    st = tf.Stream()
    for _ in range(args.warmup):
        step(st)
    st.synchronize()
    tf.device_synchronize()
    e0, e1 = tf.Event(), tf.Event()
    t0 = time.perf_counter()
    e0.record(st)
    for _ in range(args.steps):
        step(st)
    e1.record(st)
    st.synchronize()
    tf.device_synchronize()
    wall = time.perf_counter() - t0
    dev_ms = e0.elapsed_ms(e1) / args.steps   # HIP events on the launch stream
    ms_per_step = wall * 1e3 / args.steps

    flops = w.flops(cfg)
    alg_bytes = w.algorithmic_bytes(cfg)
    gflops = flops / (ms_per_step * 1e-3) / 1e9
    achieved = alg_bytes / (dev_ms * 1e-3) / 1e9
    # long rows: chunk kernel + sums, or (by column partition) hot segments, cold segments, group sums, row sums
    # (the values of the uploaded matrix are put in segment order by one more kernel on the first call only)
    n_kernels = 1 + (1 if info["n_remainder_rows"] - info["n_long_rows"] > 0 else 0) + \
        ((4 if info["long_row_hot_cols"] else 2) if info["n_long_rows"] else 0)

    check = None
    if not args.no_check:
        got = D.to_numpy()
        if op == tf.OP_SPMM_SPMM:
            t = cfg["B"].astype(np.float64) @ cfg["C"].astype(np.float64)
        else:
            t = cfg["B"].astype(np.float64) @ cfg["C"].astype(np.float64)
        want = A.astype(np.float64) @ t
        check = float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))
        if not check <= 1e-4:
            print(f"bench.py: result check failed, rel err {check:.3e}", file=sys.stderr)
            sys.exit(1)

    out = {
        "metric": METRIC, "value": round(gflops, 2), "unit": "GFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": cfg["name"], "op": cfg["op"], "rows": int(A.shape[0]), "nnz": int(A.nnz), "N": N, "K": K,
                   "lds_bytes": info["lds_bytes"], "windowed": bool(info["windowed"]), "wide_strips": bool(info["wide_strips"]), "long_row_hot_cols": info["long_row_hot_cols"], "streamed": bool(info["streamed"]), "tiles": info["n_tiles"], "fused_rows": info["n_fused_rows"],
                   "remainder_rows": info["n_remainder_rows"], "recomputed_rows": info["n_producer_rows"] - A.shape[1],
                   "writeback_rows": info["n_writeback_rows"], "kernels_per_step": n_kernels,
                   "inspector_s": round(inspect_s, 4), **({"reorder_s": round(reorder_s, 4)} if reorder_s is not None else {}), "rel_err_vs_f64": check, "device": dev["arch"]},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "algorithmic_bytes": int(alg_bytes), "kernel_ms": round(dev_ms, 5),
                     "kernel": ("fused_spmm_spmm_window64_kernel" if info["wide_strips"] else
                                "fused_spmm_spmm_window_kernel" if info["windowed"] else
                                "fused_spmm_spmm_kernel" if info["n_fused_rows"] else "spmm_rows_kernel (twice)")
                     if op == tf.OP_SPMM_SPMM else ("gemm_rows_kernel + spmm_rows_kernel" if args.unfused or info["n_fused_rows"] == 0 else
                                                    "fused_gemm_spmm_stream_kernel" if info["streamed"] else "fused_gemm_spmm_kernel"),
                     "note": "kernel_ms = HIP-event time on the launch stream / steps (all kernels of a step)"},
    }
    try:  # measured HBM traffic of the dominant kernel, if a committed profile covers this schedule
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            t = json.load(f).get(f"cfg{args.config}")
        if t and t["kernel"] == out["roofline"]["kernel"] and t["tiles"] == info["n_tiles"]:
            out["roofline"]["traffic"] = t["fetch_bytes"] + t["write_bytes"]
            out["roofline"]["traffic_source"] = t["source"]
    except (OSError, ValueError, KeyError):
        pass
    if op == tf.OP_GEMM_SPMM:
        gemm_flops = 2.0 * A.shape[1] * K * N
        out["roofline"]["mfma_frac_if_gemm_only"] = round(gemm_flops / (dev_ms * 1e-3) / 1e12 / MFMA_FP32_PEAK_TF, 4)
    if args.host_buffers:  # PCIe-inclusive: every operand crosses the bus each step
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
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
