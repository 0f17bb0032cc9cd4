#!/usr/bin/env python3
"""Benchmark of the hybrid SpMV hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload 2] [--all] [--no-sweep]

A step is one y = A*x over the whole matrix, inputs resident in HBM.  The default workload is
the FP64 block-clustered 65536x65536 matrix (synthetic workload 2) with (tau_c, tau_r) picked
by a sweep of the 5x5 grid {0,.25,.5,.75,1}^2 restricted to tau_c >= tau_r; `--all` adds the
other workloads (3: FP64 stencil, 4/5: FP16) as extra records in the same JSON line.

Prints ONE JSON line: whole-job GFLOP/s = 2*nnz/t, the roofline record of the dominant kernel
(algorithmic bytes of that kernel / its mean launch time by HIP events on the launch stream,
against 8 TB/s), and the CPU baseline (the oracle's single-thread CSR SpMV on the same matrix).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "SpMV GFLOP/s (2·nnz/t) + % of HBM roofline, FP64 and FP16, 1 GPU"
HBM_PEAK = 8.0e12  # bytes/s, MI355X HBM3E
GRID = (0.0, 0.25, 0.5, 0.75, 1.0)
# HBM-side bytes per launch (read + written) of the dominant kernels, from rocprofv3 --pmc FETCH_SIZE and
# --pmc WRITE_SIZE runs of this script, each counter scaled by what it reads for an elementwise kernel of
# known size (--calibrate-copy): FETCH_SIZE x 2.000, WRITE_SIZE x 1.000.  The text files under profiles/
# hold the counter values.  (workload, kernel, plan has tiles) -> bytes
TRAFFIC = {
    (2, "csr_rows_kernel<f64>", False): 47165962,
    (2, "csr_slice_kernel<f64>", False): 48823291,
    (3, "csr_rows_kernel<f64>", False): 287431623,
    (3, "csr_rows_kernel<f64,dict>", False): 101747762,   # one byte per value: the stencil has two distinct values
    (3, "csr_slice_kernel<f64,dict>", False): 109970561,
    (4, "csr_slice_kernel<f16>", False): 55821536,
    (5, "csr_slice_kernel<f16>", False): 301417778,
    (5, "csr_slice_kernel<f16>", True): 190181456,   # tau=(1,1): the strips run through tile_dense_kernel
}
WORKLOADS = {
    1: "configs[0]: FP64 random 4096x4096, 16 nnz/row",
    2: "configs[1]: FP64 block-clustered 65536x65536, ~64 nnz/row, 40% of nnz in dense 8x8 blocks in a 2048-wide band",
    3: "configs[2]: FP64 27-point stencil on a 100^3 grid",
    4: "configs[3]: FP16 power-law 1048576x1048576, Zipf(1.6) row lengths in [1,4096], mean ~10",
    5: "configs[4]: FP16 mixed 4194304x4194304, 20% of rows in dense 32-column strips + power-law rows",
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def kernel_bytes(mx, dtype, rows, cols, nnz):
    """Algorithmic bytes of a CSR-form SpMV over `nnz` entries (data_origin1 of the reference)."""
    return mx.algorithmic_bytes(dtype, rows, cols, nnz)


def measure(mx, torch, A, xd, yd, tau, warm, iters, flags=None):
    part = mx.Partition(A, *tau)
    plan = mx.Plan(part, mx.MX_PLAN_DEFAULT if flags is None else flags)
    tot, tile, csr = plan.time(xd, yd, warm=warm, iters=iters)
    rec = {"tau_c": tau[0], "tau_r": tau[1], "ms_total": tot, "ms_tile": tile, "ms_csr": csr,
           "tile_nnz": plan.info["tile_nnz"], "csr_nnz": plan.info["csr_nnz"],
           "tile_chunks": plan.info["tile_chunks"], "tile_bytes": plan.info["tile_bytes"],
           "csr_bytes": plan.info["csr_bytes"], "tc_nnz_ratio": part.tc_nnz_ratio if tau != (0.0, 0.0) else 0.0}
    return part, plan, rec


def run_workload(mx, torch, ora, cfg, steps, warmup, sweep, cpu_baseline, only_tau=None):
    import numpy as np
    t0 = time.time()
    A, x = mx.gen_config(cfg)
    log("workload %d: rows=%d nnz=%d generated in %.1fs" % (cfg, A.rows, A.nnz, time.time() - t0))
    dev = torch.device("cuda:0")
    xd = torch.from_numpy(x).to(dev)
    yd = torch.empty(A.rows, dtype=xd.dtype, device=dev)
    B = A.algorithmic_bytes
    dtype = "f64" if A.dtype == mx.MX_F64 else "f16"

    # tau sweep with short timing loops
    points = [(c, r) for c in GRID for r in GRID if c >= r] if sweep else [(0.0, 0.0)]
    if only_tau is not None:
        points = [tuple(only_tau)]  # nothing else: a profile of this run then shows one plan's kernels only
    table = []
    # (MX_PLAN_KEEP_TILES: every point runs the hybrid its fragments give, also where the plan's own
    # estimate would send everything through the CSR part; what that estimate says is recorded below)
    for tau in points:
        part, plan, rec = measure(mx, torch, A, xd, yd, tau, 20, 200, mx.MX_PLAN_KEEP_TILES)
        table.append(rec)
        log("  tau=(%.2f,%.2f) total %.2f us (tile %.2f + csr %.2f) tile_nnz=%d" %
            (tau[0], tau[1], rec["ms_total"] * 1e3, rec["ms_tile"] * 1e3, rec["ms_csr"] * 1e3, rec["tile_nnz"]))
        plan.close()
        part.close()
    best = min(table, key=lambda r: r["ms_total"]) if only_tau is None else table[-1]
    if best["tile_nnz"] == 0 and only_tau is None:
        # every point that sends nothing to the tile kernel is the same CSR-only plan: call it (0, 0)
        best = next(r for r in table if (r["tau_c"], r["tau_r"]) == (0.0, 0.0))
    hybrid = [r for r in table if r["tile_nnz"] > 0]
    best_hybrid = min(hybrid, key=lambda r: r["ms_total"]) if hybrid else None
    csr_only = next((r for r in table if (r["tau_c"], r["tau_r"]) == (0.0, 0.0)), None)

    # the timed run on the best point: W warm-up steps, then exactly K steps between syncs
    tau = (best["tau_c"], best["tau_r"])
    if best_hybrid:
        p2 = mx.Partition(A, best_hybrid["tau_c"], best_hybrid["tau_r"])
        q2 = mx.Plan(p2)  # default flags: the plan's own decision at the best hybrid point
        best_hybrid["default_plan_keeps_tiles"] = q2.info["tile_nnz"] > 0
        q2.close()
        p2.close()
    part, plan, _ = measure(mx, torch, A, xd, yd, tau, 5, 20, mx.MX_PLAN_KEEP_TILES)
    plan.spmv_repeat(xd, yd, warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    plan.spmv_repeat(xd, yd, steps)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    # per-kernel launch durations by HIP events on the plan's own stream
    ev_total, ev_tile, ev_csr = plan.time(xd, yd, warm=warmup, iters=steps)
    y = yd.cpu().numpy().astype(np.float64)

    # parity of the timed configuration against the oracle
    if A.dtype == mx.MX_F64:
        ref = ora.spmv_f64(A.val, A.rowPtr, A.colInd, x)
    else:
        ref = ora.spmv_f16_f32acc(A.val, A.rowPtr, A.colInd, x)[0].astype(np.float64)
    rel_l2 = float(np.linalg.norm(y - ref) / np.linalg.norm(ref))

    # the same SpMV with cold caches: a 1 GiB buffer is swept between launches, so neither the
    # L2s (8 x 4 MB) nor the 256 MB memory-side cache hold the matrix when the launch starts
    flush = torch.empty(1 << 28, dtype=torch.float32, device=dev)
    cold = []
    for _ in range(15):
        flush.add_(1.0)
        torch.cuda.synchronize()
        cold.append(plan.time(xd, yd, warm=0, iters=1, parts=False)[0])
    del flush
    cold_ms = float(np.median(cold))

    info = plan.info
    if ev_tile > ev_csr:
        dom = {"kernel": "tile_%s_kernel" % dtype, "ms": ev_tile,
               "bytes": kernel_bytes(mx, A.dtype, min(A.rows, 8 * info["tile_chunks"]), 0, info["tile_nnz"])}
    else:
        # the CSR part's main kernel alone (the slice variant has a small combine kernel after it)
        ms_main = plan.time_csr_main(xd, yd, warm=warmup, iters=steps)
        name = "csr_slice_kernel<%s>" if info["csr_main_kernel"] == 1 else "csr_rows_kernel<%s>"
        if info["csr_value_dict"]:
            name = name.replace("<%s>", "<%s,dict>")
        dom = {"kernel": name % dtype, "ms": ms_main,
               "bytes": kernel_bytes(mx, A.dtype, A.rows, A.cols, info["csr_main_nnz"])}
    achieved = dom["bytes"] / (dom["ms"] * 1e-3)
    rec = {
        "workload": WORKLOADS[cfg], "dtype": dtype, "rows": A.rows, "nnz": A.nnz,
        "tau_c": tau[0], "tau_r": tau[1], "csr_variant": ("rows", "slices", "split")[info["csr_variant"]],
        "ms_per_step": wall_ms, "ms_per_step_events": ev_total,
        "gflops": 2.0 * A.nnz / (wall_ms * 1e-3) / 1e9,
        "algorithmic_bytes": B,
        "hbm_frac_whole_spmv": B / (wall_ms * 1e-3) / HBM_PEAK,
        "cold_cache": {"ms_per_step": cold_ms, "gflops": 2.0 * A.nnz / (cold_ms * 1e-3) / 1e9,
                       "hbm_frac_whole_spmv": B / (cold_ms * 1e-3) / HBM_PEAK,
                       "how": "median of 15 single launches, each after a 1 GiB buffer sweep and a sync; "
                              "the quoted value is the back-to-back (warm) one"},
        "rel_l2_vs_oracle": rel_l2,
        "csr_only_ms": csr_only and csr_only["ms_total"],
        "best_hybrid": best_hybrid and {k: best_hybrid[k] for k in ("tau_c", "tau_r", "ms_total", "tile_nnz", "csr_nnz", "default_plan_keeps_tiles")},
        "roofline": {"bound": "hbm", "kernel": dom["kernel"], "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK,
                     "traffic": TRAFFIC.get((cfg, dom["kernel"], info["tile_nnz"] > 0)),
                     "bytes_per_launch": dom["bytes"], "ms_per_launch": dom["ms"],
                     **({"note": "the matrix has %d distinct values and the kernel reads one byte per entry for them: the "
                                 "algorithmic bytes still count sizeof(valT) per entry, so frac can exceed 1; `traffic` is "
                                 "what the kernel really moves" % info["csr_value_dict"]} if info["csr_value_dict"] else {})},
        "sweep": [{k: r[k] for k in ("tau_c", "tau_r", "ms_total", "ms_tile", "ms_csr", "tile_nnz")} for r in table],
    }
    if cpu_baseline:
        reps = []
        runner = (lambda: ora.spmv_f64(A.val, A.rowPtr, A.colInd, x)) if A.dtype == mx.MX_F64 else \
                 (lambda: ora.spmv_f16_f32acc(A.val, A.rowPtr, A.colInd, x))
        # one thread on one core, as the reference's spmv_serial: pinned for the duration
        affinity = os.sched_getaffinity(0)
        pinned = None
        try:
            pinned = min(affinity)
            os.sched_setaffinity(0, {pinned})
        except OSError:
            pinned = None
        try:
            for i in range(12):
                t0 = time.perf_counter()
                runner()
                reps.append(time.perf_counter() - t0)
        finally:
            if pinned is not None:
                os.sched_setaffinity(0, affinity)
        t_cpu = min(reps[2:])
        cpu_model = "unknown"
        try:
            with open("/proc/cpuinfo") as f:
                cpu_model = next((l.split(":", 1)[1].strip() for l in f if l.startswith("model name")), "unknown")
        except OSError:
            pass
        rec["cpu_baseline"] = {"value": 2.0 * A.nnz / t_cpu / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": "port",
                               "cpu": cpu_model, "cpus_visible": len(os.sched_getaffinity(0)), "pinned_to_cpu": pinned,
                               "sample": "the full matrix of this workload, best of 10 after 2 warm-ups "
                                         "(%.1f ms per SpMV), single thread as the reference's spmv_serial" % (t_cpu * 1e3)}
        # not the reference's: the same oracle routine over nnz-balanced row ranges, one thread per
        # core (the C call releases the interpreter lock)
        from concurrent.futures import ThreadPoolExecutor
        ncore = max(1, min(16, len(os.sched_getaffinity(0))))
        cuts = np.searchsorted(A.rowPtr, np.linspace(0, A.nnz, ncore + 1)).astype(int)
        cuts[0], cuts[-1] = 0, A.rows
        f16 = A.dtype != mx.MX_F64

        def part_run(k):
            r0, r1 = int(cuts[k]), int(cuts[k + 1])
            if r1 > r0:
                (ora.spmv_f16_f32acc if f16 else ora.spmv_f64)(A.val, A.rowPtr[r0:r1 + 1], A.colInd, x)
        reps = []
        with ThreadPoolExecutor(ncore) as ex:
            for i in range(7):
                t0 = time.perf_counter()
                list(ex.map(part_run, range(ncore)))
                reps.append(time.perf_counter() - t0)
        t_all = min(reps[2:])
        rec["cpu_all_cores"] = {"value": 2.0 * A.nnz / t_all / 1e9, "unit": "GFLOP/s", "cores": ncore, "kind": "port",
                                "sample": "not the reference's (its CPU path is serial): the oracle routine on %d "
                                          "nnz-balanced row ranges in parallel threads, best of 5 (%.2f ms)" % (ncore, t_all * 1e3)}
        # the extraction itself (not part of `value`): host route against the device route, same partition
        pt = (0.5, 0.25)
        mx.Partition(A, *pt, device=True).close()  # first use of the device code
        t0 = time.perf_counter()
        ph = mx.Partition(A, *pt)
        t1 = time.perf_counter()
        pd = mx.Partition(A, *pt, device=True)
        t2 = time.perf_counter()
        rec["preprocess"] = {"tau_c": pt[0], "tau_r": pt[1], "host_ms": (t1 - t0) * 1e3, "device_route_ms": (t2 - t1) * 1e3,
                             "same_partition": ph.hash == pd.hash,
                             "note": "mx_partition_create on the host cores against mx_partition_create_device "
                                     "(upload, extraction on the GPU, download)"}
        ph.close()
        pd.close()
    plan.close()
    part.close()
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=4000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", type=int, default=2, choices=sorted(WORKLOADS))
    ap.add_argument("--all", action="store_true", help="also run workloads 3, 4, 5 (reported under 'others')")
    ap.add_argument("--no-sweep", action="store_true", help="tau=(0,0) only")
    ap.add_argument("--tau", type=float, nargs=2, metavar=("TAU_C", "TAU_R"), default=None,
                    help="no sweep: run this point (a profile of a fixed plan)")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="also launch one elementwise kernel that reads and writes MIB MiB (a known size to "
                         "scale rocprofv3's FETCH_SIZE / WRITE_SIZE counters by)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on exactly one GPU (the hybrid SpMV path has no multi-GPU part); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    import matxtractt_amd as mx
    from oracle import mx_oracle as ora
    if not torch.cuda.is_available() or mx.device_count() < 1:
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(1)

    main_rec = run_workload(mx, torch, ora, args.workload, args.steps, args.warmup, not args.no_sweep, True, args.tau)
    out = {
        "metric": METRIC, "value": main_rec["gflops"], "unit": "GFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": main_rec["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": main_rec["dtype"], "data": "synthetic",
        "config": {"workload": main_rec["workload"], "rows": main_rec["rows"], "nnz": main_rec["nnz"],
                   "tau_c": main_rec["tau_c"], "tau_r": main_rec["tau_r"], "csr_variant": main_rec["csr_variant"],
                   "tau_grid": "5x5 {0,.25,.5,.75,1}^2, tau_c>=tau_r, best of sweep" if args.tau is None and not args.no_sweep
                   else "no sweep: point fixed on the command line"},
        "roofline": main_rec["roofline"],
        "cpu_baseline": main_rec.pop("cpu_baseline"),
        "cpu_all_cores": main_rec.pop("cpu_all_cores"),
        "preprocess": main_rec.pop("preprocess"),
        "hbm_frac_whole_spmv": main_rec["hbm_frac_whole_spmv"],
        "cold_cache": main_rec["cold_cache"],
        "rel_l2_vs_oracle": main_rec["rel_l2_vs_oracle"],
        "csr_only_ms": main_rec["csr_only_ms"],
        "best_hybrid": main_rec["best_hybrid"],
        "sweep": main_rec["sweep"],
    }
    # what a plain device copy reaches on this GPU, next to the 8 TB/s the roofline is priced at:
    # read + written bytes over the time of back-to-back copies, at this workload's algorithmic
    # size and at 1 GiB
    copy = {}
    for label, nbytes in (("workload_sized", int(main_rec["roofline"]["bytes_per_launch"]) // 2), ("1GiB", 1 << 29)):
        src = torch.ones(nbytes // 4, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = 200 if nbytes < (1 << 27) else 20
        e0.record()
        for _ in range(reps):
            dst.copy_(src)
        e1.record()
        torch.cuda.synchronize()
        copy[label] = {"bytes_read_plus_written": 2 * (nbytes // 4) * 4, "GBs": 2 * (nbytes // 4) * 4 / (e0.elapsed_time(e1) / reps * 1e-3) / 1e9}
        del src, dst
    out["device_copy"] = copy
    if args.calibrate_copy:
        n = args.calibrate_copy * (1 << 20) // 4
        src = torch.ones(n, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)  # reads 4n bytes, writes 4n bytes
        torch.cuda.synchronize()
        out["calibrate_copy_bytes_each_way"] = 4 * n
    if args.all:
        others = {}
        for cfg in (3, 4, 5):
            if cfg == args.workload:
                continue
            r = run_workload(mx, torch, ora, cfg, max(200, args.steps // 4), args.warmup, not args.no_sweep, False)
            others["workload_%d" % cfg] = {k: r[k] for k in (
                "workload", "dtype", "rows", "nnz", "tau_c", "tau_r", "csr_variant", "ms_per_step", "gflops", "hbm_frac_whole_spmv",
                "cold_cache", "rel_l2_vs_oracle", "csr_only_ms", "best_hybrid", "roofline")}
        out["others"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
