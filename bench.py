#!/usr/bin/env python3
"""Benchmark of the hybrid SpMV hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload N ...] [--no-sweep | --tau C R]

A step is one y = A*x over the whole matrix, inputs resident in HBM.  With no flags the four
GPU workloads of the benchmark run: the headline is the largest one, workload 5 (FP16 mixed,
4.2 M rows, 63 M entries; (tau_c, tau_r) = best of the 5x5 grid {0,.25,.5,.75,1}^2 with
tau_c >= tau_r), and workloads 2 (FP64 block-clustered, same sweep), 3 (FP64 stencil) and 4
(FP16 power-law) follow under "others", each with its own roofline record, parity figure and
cold-cache time.

Prints ONE JSON line.  `value` = 2*nnz/t of the headline workload (GFLOP/s), timed on the plan a
caller gets with default flags at the best point of the sweep (the sweep itself keeps every
hybrid's tiles, so that its table shows each one as it is).  `roofline` prices the WHOLE product:
the reference's algorithmic bytes of the matrix (nnz*(sizeof(valT)+4) + (rows+1)*4 +
cols*sizeof(valT) + rows*sizeof(valT), test/test_cdspmv.cpp:214) over the time of one product
against 8 TB/s.  Three times are measured, each the median of five repetitions of the
reference's protocol (200 warm-ups, then at least 1000 timed launches between HIP events on the
plan's own stream, src/spmv_kernel/cdSpMV.cu:454-479): `warm` (one plan, back to back: a matrix
of up to 256 MB stays in the memory-side cache), `rotating` (a train that takes several copies
of the plan in turn, three times the memory-side cache in all: every array comes from HBM, the
steady state of a solver whose matrix does not fit that cache) and `cold` (single products after
a 1 GiB sweep).  `roofline.frac` is the warm figure for a plan that fits the memory-side cache
(by the bytes a product touches as the plan stores them, `plan_bytes_per_product`) and the
rotating one for a plan that does not (`frac_basis` says which; all three are there),
and `frac_traffic` prices the same time with the bytes the counters saw instead of the
algorithmic ones.  `csr_entries_kept_in_cache` says how the plan reads the entries of its slices
(plain loads, so that a matrix that fits the L2s or the memory-side cache stays there between
products, or streaming loads: the plan's own choice by size, mx_plan_info.csr_keep).  `roofline.kernels` lists every kernel launch of the product timed alone, each
with its share of the algorithmic bytes (the shares add up to the whole) and, where profiles/
holds a rocprofv3 counter run of that kernel on that workload and plan, its measured HBM
traffic.  `cpu_baseline` is the oracle's single-thread CSR loop on the same matrix, on this
box's host cores.  Workloads 2 and 5 are also run with their dense structure off the grid of
eight columns (`others.workload_N_unaligned`: CSR-only against the best hybrid).
"""
import argparse
import glob
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "SpMV GFLOP/s (2·nnz/t) + % of HBM roofline, FP64 and FP16, 1 GPU"
HBM_PEAK = 8.0e12  # bytes/s, MI355X HBM3E
MALL_BYTES = 256 << 20  # the memory-side cache
REPS = 5  # repetitions of every timed train; the median is quoted
GRID = (0.0, 0.25, 0.5, 0.75, 1.0)
WORKLOADS = {
    1: "configs[0]: FP64 random 4096x4096, 16 nnz/row",
    2: "configs[1]: FP64 block-clustered 65536x65536, ~64 nnz/row, 40% of nnz in dense 8x8 blocks in a 2048-wide band",
    3: "configs[2]: FP64 27-point stencil on a 100^3 grid",
    4: "configs[3]: FP16 power-law 1048576x1048576, Zipf(1.6) row lengths in [1,4096], mean ~10",
    5: "configs[4]: FP16 mixed 4194304x4194304, 20% of rows in dense 32-column strips + power-law rows",
}
SWEPT = (2, 5)  # the workloads whose 5 x 5 grid of extraction fractions is swept; 3 and 4 run CSR-only and at two hybrid points for the record


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def read_traffic():
    """HBM bytes per launch from the rocprofv3 counter runs under profiles/: lines of the form
    `TRAFFIC workload=<n> plan=<csr_only|hybrid> kernel=<name> read=<bytes> written=<bytes>` (FETCH_SIZE and
    WRITE_SIZE per dispatch, scaled by what the same counters read for a copy kernel of known size;
    the files say how).  Nothing is hard-coded here: a kernel without such a line reports null."""
    table = {}
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.txt"))):
        with open(path) as f:
            for line in f:
                m = re.match(r"TRAFFIC workload=(\d+) plan=(\w+) kernel=(\S+) read=(\d+) written=(\d+)", line.strip())
                if m:
                    table[(int(m.group(1)), m.group(2), m.group(3))] = {
                        "read": int(m.group(4)), "written": int(m.group(5)), "file": os.path.relpath(path, ROOT)}
    return table


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            return next((l.split(":", 1)[1].strip() for l in f if l.startswith("model name")), "unknown")
    except OSError:
        return "unknown"


def cpu_baseline(mx, ora, A, x):
    """The oracle's CSR loop on the same matrix: one thread pinned to one core, as the reference's
    spmv_serial; and (labelled as not the reference's) the same routine on all cores."""
    import numpy as np
    f16 = A.dtype != mx.MX_F64
    run = (lambda rp: ora.spmv_f16_f32acc(A.val, rp, A.colInd, x)) if f16 else (lambda rp: ora.spmv_f64(A.val, rp, A.colInd, x))
    affinity = os.sched_getaffinity(0)
    pinned = None
    try:
        pinned = min(affinity)
        os.sched_setaffinity(0, {pinned})
    except OSError:
        pinned = None
    reps = []
    try:
        for _ in range(12):
            t0 = time.perf_counter()
            run(A.rowPtr)
            reps.append(time.perf_counter() - t0)
    finally:
        if pinned is not None:
            os.sched_setaffinity(0, affinity)
    t_cpu = min(reps[2:])
    base = {"value": 2.0 * A.nnz / t_cpu / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": "port",
            "cpu": cpu_model(), "cpus_visible": len(affinity), "pinned_to_cpu": pinned,
            "sample": "the full matrix of the headline workload, best of 10 after 2 warm-ups (%.1f ms per SpMV, %.1f s of "
                      "CPU work in all), single thread as the reference's spmv_serial" % (t_cpu * 1e3, sum(reps))}
    from concurrent.futures import ThreadPoolExecutor
    ncore = max(1, min(16, len(affinity)))
    cuts = np.searchsorted(A.rowPtr, np.linspace(0, A.nnz, ncore + 1)).astype(int)
    cuts[0], cuts[-1] = 0, A.rows

    def part_run(k):
        r0, r1 = int(cuts[k]), int(cuts[k + 1])
        if r1 > r0:
            run(A.rowPtr[r0:r1 + 1])
    reps = []
    with ThreadPoolExecutor(ncore) as ex:
        for _ in range(7):
            t0 = time.perf_counter()
            list(ex.map(part_run, range(ncore)))
            reps.append(time.perf_counter() - t0)
    t_all = min(reps[2:])
    allc = {"value": 2.0 * A.nnz / t_all / 1e9, "unit": "GFLOP/s", "cores": ncore, "kind": "port",
            "sample": "not the reference's (its CPU path is serial): the oracle routine on %d nnz-balanced row ranges in "
                      "parallel threads, best of 5 (%.2f ms)" % (ncore, t_all * 1e3)}
    return base, allc


def median_time(fn, reps=REPS):
    import numpy as np
    return float(np.median([fn() for _ in range(reps)]))


def run_workload(mx, torch, ora, cfg, steps, warmup, mode, traffic, only_tau=None, keep=None, unaligned=False, brief=False, scale=1.0, timed_flags=None):
    """mode: 'sweep' (the 5x5 grid), 'points' (CSR-only and two hybrid points) or 'csr' ((0,0) only).
    brief: no routes, no cold or rotating trains (the records of the unaligned variants)."""
    import numpy as np
    keep = mx.MX_PLAN_KEEP_TILES if keep is None else keep
    t0 = time.time()
    A, x = mx.gen_config(cfg, scale=scale, unaligned=unaligned)
    log("workload %d%s: rows=%d nnz=%d generated in %.1fs" % (cfg, " (off the grid)" if unaligned else "", A.rows, A.nnz, time.time() - t0))
    dev = torch.device("cuda:0")
    xd = torch.from_numpy(x).to(dev)
    yd = torch.empty(A.rows, dtype=xd.dtype, device=dev)
    B = A.algorithmic_bytes
    dtype = "f64" if A.dtype == mx.MX_F64 else "f16"
    n_ev = max(steps, 1000)
    on_device = A.nnz >= (1 << 21)

    # ---- which (tau_c, tau_r): every candidate is partitioned (on the device for large matrices),
    # planned and timed by mx_tune_tau with short loops; candidates that send nothing to the tile
    # kernels are one and the same CSR-only plan and are timed once.  MX_PLAN_KEEP_TILES: every
    # candidate runs the hybrid its fragments give, also where the plan's own estimate would send
    # everything through the CSR part.  The three fastest candidates and the CSR-only plan are then
    # timed again with the full protocol, and the point is chosen from those.
    t0 = time.time()
    if only_tau is not None:
        points = [tuple(only_tau)]
    elif mode == "sweep":
        points = None
    elif mode == "points":
        points = [(0.0, 0.0), (0.5, 0.25), (1.0, 1.0)]
    else:
        points = [(0.0, 0.0)]
    table = []
    if points is None:
        _, _, tt = mx.tune_tau(A, levels=5, flags=keep, warm=10, iters=100)
        table = [{"tau_c": c, "tau_r": r, "ms_total": ms, "tile_nnz": tn} for c, r, ms, tn in tt]
    else:
        for tau in points:
            part = mx.Partition(A, *tau, device=on_device and tau != (0.0, 0.0))
            plan = mx.Plan(part, keep)
            ms = plan.time(xd, yd, warm=10, iters=100, parts=False)[0]
            table.append({"tau_c": tau[0], "tau_r": tau[1], "ms_total": ms, "tile_nnz": plan.info["tile_nnz"]})
            plan.close()
            part.close()
    csr_rec = next((r for r in table if r["tile_nnz"] == 0), None)
    again = sorted((r for r in table if r["tile_nnz"] > 0), key=lambda r: r["ms_total"])[:3]
    if csr_rec is not None:
        again.append(csr_rec)
    for r in again:
        part = mx.Partition(A, r["tau_c"], r["tau_r"], device=on_device and r["tile_nnz"] > 0)
        plan = mx.Plan(part, keep)
        r["ms_short_loop"] = r["ms_total"]
        r["ms_total"] = median_time(lambda: plan.time(xd, yd, warm=200, iters=1000, parts=False)[0], 3)
        r["timed"] = "median of 3 x (200 + 1000)"
        plan.close()
        part.close()
    for r in table:
        log("  tau=(%.2f,%.2f) %.2f us tile_nnz=%d%s" % (r["tau_c"], r["tau_r"], r["ms_total"] * 1e3, r["tile_nnz"],
                                                         "  (timed again)" if "timed" in r else ""))
    sweep_s = time.time() - t0
    csr_only = csr_rec
    hybrid = [r for r in table if r["tile_nnz"] > 0 and "timed" in r]
    best_hybrid = min(hybrid, key=lambda r: r["ms_total"]) if hybrid else None
    best = min((r for r in table if "timed" in r), key=lambda r: r["ms_total"])
    # a hybrid point is taken when it beats the CSR-only plan by more than 2 %; every point without tiles is
    # the CSR-only plan: call it (0, 0)
    if csr_only is not None and (best["tile_nnz"] == 0 or best["ms_total"] > 0.98 * csr_only["ms_total"]):
        best = dict(csr_only, tau_c=0.0, tau_r=0.0)
    tau = (best["tau_c"], best["tau_r"])

    # ---- the plan of the best point as a caller with default flags gets it, from the matrix to the first y:
    # host route and device route
    FLAGS = timed_flags if timed_flags is not None else mx.MX_PLAN_DEFAULT if keep == mx.MX_PLAN_KEEP_TILES else keep

    def first_y(device):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        part = mx.Partition(A, *tau, device=device)
        t1 = time.perf_counter()
        plan = mx.Plan(part, FLAGS)
        t2 = time.perf_counter()
        plan.spmv(xd, yd)
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        return part, plan, {"partition_ms": (t1 - t0) * 1e3, "plan_create_ms": (t2 - t1) * 1e3,
                            "first_spmv_ms": (t3 - t2) * 1e3, "total_ms": (t3 - t0) * 1e3}
    # "host": what a caller of the reference's surface gets (matxtract_preprocess + mx_plan_create, host arrays in):
    # the extraction on the GPU for a matrix of two million entries or more, the plan from the partition's device arrays
    part, plan, host_route = first_y(None)
    route = {"host": host_route}
    info = plan.info
    if not brief:
        # the device route: the matrix goes up as it is; extraction, decisions and layouts are made on the device from
        # the device arrays (mx_plan_create_device: the same plan, so the same y bit for bit); a caller whose matrix
        # already lives in HBM skips the upload
        if not getattr(run_workload, "_device_route_used", False):
            A1 = mx.gen_config(1)[0]  # first use of the device code, not timed
            mx.Plan.from_device(*(torch.from_numpy(a).to(dev) for a in (A1.rowPtr, A1.colInd, A1.val)), A1.cols, 0.5, 0.5).close()
            run_workload._device_route_used = True
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        drp, dci, dva = (torch.from_numpy(a).to(dev) for a in (A.rowPtr, A.colInd, A.val))
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        q2 = mx.Plan.from_device(drp, dci, dva, A.cols, tau[0], tau[1], FLAGS)
        t2 = time.perf_counter()
        y2 = torch.empty_like(yd)
        q2.spmv(xd, y2)
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        route["device"] = {"upload_ms": (t1 - t0) * 1e3, "plan_create_ms": (t2 - t1) * 1e3, "first_spmv_ms": (t3 - t2) * 1e3,
                           "total_ms": (t3 - t0) * 1e3, "prep_route": q2.info["prep_route"]}
        route["same_y"] = bool(torch.equal(y2, yd))
        q2.close()
        del drp, dci, dva, y2

    # ---- the timed run: W warm-up products, then exactly K products between synchronisations
    plan.spmv_repeat(xd, yd, warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    plan.spmv_repeat(xd, yd, steps)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    # the reference's protocol: warm-ups, then a train of launches between HIP events on the plan's own stream;
    # the median of REPS such trains
    ev_total = median_time(lambda: plan.time(xd, yd, warm=max(warmup, 200), iters=n_ev, parts=False)[0])
    kernels = plan.time_kernels(xd, yd, warm=max(warmup, 100), iters=n_ev)
    y = yd.cpu().numpy().astype(np.float64)

    # ---- parity of the timed configuration against the oracle
    if A.dtype == mx.MX_F64:
        ref = ora.spmv_f64(A.val, A.rowPtr, A.colInd, x)
    else:
        ref = ora.spmv_f16_f32acc(A.val, A.rowPtr, A.colInd, x)[0].astype(np.float64)
    rel_l2 = float(np.linalg.norm(y - ref) / np.linalg.norm(ref))

    # what one product touches as the plan stores it (a value dictionary stores a byte where the algorithmic count has the
    # value): that, not the algorithmic count, is what has to fit the memory-side cache
    plan_bytes = info["touched_bytes"]
    cold_ms = rot = None
    if not brief:
        # ---- cold caches: a 1 GiB buffer is swept between launches, so neither the L2s (8 x 4 MB) nor
        # the 256 MB memory-side cache hold the matrix when the product starts
        flush = torch.empty(1 << 28, dtype=torch.float32, device=dev)
        cold = []
        for _ in range(15):
            flush.add_(1.0)
            torch.cuda.synchronize()
            cold.append(plan.time(xd, yd, warm=0, iters=1, parts=False)[0])
        del flush
        cold_ms = float(np.median(cold))
        # ---- every array from HBM, in a steady train: copies of the plan (and of x and y), three times the
        # memory-side cache in all, taken in turn
        copies = int(min(24, max(2, -(-3 * MALL_BYTES // max(int(plan_bytes), 1)))))
        plans, xs, ys = [plan], [xd], [yd]
        for _ in range(copies - 1):
            plans.append(mx.Plan(part, FLAGS))
            xs.append(xd.clone())
            ys.append(torch.empty_like(yd))
        rot_ms = median_time(lambda: mx.time_rotate(plans, xs, ys, warm=max(200, 4 * copies), iters=max(n_ev, 20 * copies)))
        same = all(bool(torch.equal(ys[i], yd)) for i in range(1, copies))
        for p in plans[1:]:
            p.close()
        del plans, xs, ys
        rot = {"copies": copies, "bytes_in_rotation": copies * plan_bytes, "ms_per_step": rot_ms,
               "gflops": 2.0 * A.nnz / (rot_ms * 1e-3) / 1e9, "hbm_frac_whole_spmv": B / (rot_ms * 1e-3) / HBM_PEAK,
               "every_copy_gives_the_same_y": same,
               "how": "median of %d trains of >= %d products that take %d copies of the plan (each with its own x and y) in "
                      "turn, HIP events on one stream" % (REPS, max(n_ev, 20 * copies), copies)}

    # ---- what the plan's own estimate decides at the best hybrid point (default flags)
    if best_hybrid:
        p2 = mx.Partition(A, best_hybrid["tau_c"], best_hybrid["tau_r"], device=on_device)
        q2 = mx.Plan(p2)
        best_hybrid = dict(best_hybrid, default_plan_keeps_tiles=q2.info["tile_nnz"] > 0)
        q2.close()
        p2.close()

    plan_kind = "hybrid" if info["tile_nnz"] > 0 else "csr_only"
    krecs, tr_sum, tr_all = [], 0, True
    for k in kernels:
        t = traffic.get((cfg, plan_kind, k["name"])) if not unaligned else None
        if t is None:
            tr_all = False
        else:
            tr_sum += t["read"] + t["written"]
        krecs.append({"kernel": k["name"], "ms_per_launch": k["ms"], "nnz": k["nnz"],
                      "algorithmic_bytes": k["algorithmic_bytes"],
                      "achieved": k["algorithmic_bytes"] / (k["ms"] * 1e-3) / 1e9,
                      "frac": k["algorithmic_bytes"] / (k["ms"] * 1e-3) / HBM_PEAK,
                      "traffic": (t["read"] + t["written"]) if t else None,
                      "traffic_from": t["file"] if t else None})
    # the time the fraction is priced on: the warm train for a plan that fits the memory-side cache (a solver
    # that iterates on it finds it there), the rotating train for one that does not
    in_mall = plan_bytes <= MALL_BYTES or rot is None
    basis_ms = ev_total if in_mall else rot["ms_per_step"]
    achieved = B / (basis_ms * 1e-3)
    traffic_total = tr_sum if (tr_all and krecs) else None
    roofline = {"bound": "hbm", "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": achieved / HBM_PEAK,
                "frac_basis": ("warm: the plan's %.0f MB stay in the 256 MB memory-side cache between products" % (plan_bytes / 1e6)) if plan_bytes <= MALL_BYTES
                else ("warm: one plan back to back (no rotating train was run for this variant; its %.0f MB do not fit the memory-side cache)" % (plan_bytes / 1e6)) if rot is None
                else ("rotating: the plan's %.0f MB do not fit the 256 MB memory-side cache, every product reads them from HBM" % (plan_bytes / 1e6)),
                "frac_warm": B / (ev_total * 1e-3) / HBM_PEAK,
                "frac_rotating": rot and rot["hbm_frac_whole_spmv"],
                "frac_cold": cold_ms and B / (cold_ms * 1e-3) / HBM_PEAK,
                "traffic": traffic_total,
                "frac_traffic": traffic_total and traffic_total / (basis_ms * 1e-3) / HBM_PEAK,
                "what": "the whole product (%s): algorithmic bytes of the matrix over the median, over %d trains, of the mean time "
                        "of one product in a train of %d products after 200 warm-ups, HIP events on the plan's stream" %
                        (" + ".join(k["kernel"] for k in krecs), REPS, n_ev),
                "bytes_per_launch": B, "ms_per_launch": basis_ms, "kernels": krecs}
    if info["csr_value_dict"]:
        roofline["note"] = ("the matrix has %d distinct values and the main kernel reads one byte per entry for them: the "
                            "algorithmic bytes still count sizeof(valT) per entry, so frac can exceed 1; frac_traffic prices "
                            "the same time with the bytes the kernels really move" % info["csr_value_dict"])
    rec = {
        "workload": WORKLOADS[cfg] + (", dense structure off the grid of eight columns" if unaligned else "") +
        ("" if scale == 1.0 else ", at %g of the benchmark's rows" % scale),
        "dtype": dtype, "rows": A.rows, "nnz": A.nnz,
        "tau_c": tau[0], "tau_r": tau[1], "plan": plan_kind, "plan_flags": "MX_PLAN_DEFAULT" if FLAGS == mx.MX_PLAN_DEFAULT else "MX_PLAN_KEEP_TILES" if FLAGS == mx.MX_PLAN_KEEP_TILES else int(FLAGS),
        "csr_variant": ("rows", "slices", "split")[info["csr_variant"]], "csr_one_launch": bool(info["csr_fused"]),
        "csr_entries_kept_in_cache": bool(info["csr_keep"]),
        "tile_nnz": info["tile_nnz"], "csr_nnz": info["csr_nnz"],
        "ms_per_step": wall_ms, "ms_per_step_events": ev_total,
        "gflops": 2.0 * A.nnz / (wall_ms * 1e-3) / 1e9,
        "algorithmic_bytes": B, "plan_bytes_per_product": plan_bytes,
        "hbm_frac_whole_spmv": B / (wall_ms * 1e-3) / HBM_PEAK,
        "cold_cache": cold_ms and {"ms_per_step": cold_ms, "gflops": 2.0 * A.nnz / (cold_ms * 1e-3) / 1e9,
                                   "hbm_frac_whole_spmv": B / (cold_ms * 1e-3) / HBM_PEAK,
                                   "how": "median of 15 single products, each after a 1 GiB buffer sweep and a sync"},
        "rotating": rot,
        "rel_l2_vs_oracle": rel_l2,
        # mx_plan_create from a partition in host memory; mx_plan_create_device from the matrix in device memory,
        # extraction included (matrix_to_first_y has both routes whole)
        "plan_create_ms": host_route["plan_create_ms"],
        "plan_create_device_ms": route.get("device", {}).get("plan_create_ms"),
        "matrix_to_first_y": route,
        "plan_estimates_us": {"rows": info["est_rows_us"], "slices": info["est_slices_us"]},
        "csr_only_ms": csr_only and csr_only["ms_total"],
        "best_hybrid": best_hybrid,
        "roofline": roofline,
        "sweep": table, "sweep_flags": "MX_PLAN_KEEP_TILES" if keep == mx.MX_PLAN_KEEP_TILES else int(keep), "sweep_seconds": sweep_s,
    }
    plan.close()
    part.close()
    return rec, (A, x)


def tau_family(mx, torch, scales):
    """mx_estimate_tau held against mx_tune_tau on matrices neither was calibrated on: the families around
    workloads 5 (5 to 40 % of the row runs in strips) and 2 (10 to 70 % of the entries in 8x8 blocks), on and off
    the grid of eight columns.  Per case: the estimated and the timed fractions, the time of a default plan at
    each (median of 3 trains of 200 + 1000 products) and the regret of the estimate."""
    dev = torch.device("cuda:0")

    def timed(A, xd, tau):
        part = mx.Partition(A, tau[0], tau[1])
        plan = mx.Plan(part, mx.MX_PLAN_DEFAULT)
        y = torch.zeros(A.rows, dtype=xd.dtype, device=dev)
        ms = median_time(lambda: plan.time(xd, y, 200, 1000, parts=False)[0], 3)
        tiles = plan.info["tile_nnz"]
        plan.close()
        part.close()
        return ms, tiles
    rows = []
    for scale in scales:
        for unaligned in (False, True):
            for cfg, shares in ((5, (0.05, 0.1, 0.2, 0.4)), (2, (0.1, 0.25, 0.4, 0.7))):
                for share in shares:
                    A, x = mx.gen_config(cfg, scale=scale, unaligned=unaligned, dense_share=share)
                    xd = torch.from_numpy(x).to(dev)
                    ec, er, _ = mx.estimate_tau(A, 5)
                    tc, tr, _ = mx.tune_tau(A, 5, mx.MX_PLAN_DEFAULT, 50, 300)
                    ms_e, tiles_e = timed(A, xd, (ec, er))
                    same = (ec, er) == (tc, tr)
                    ms_t, tiles_t = (ms_e, tiles_e) if same else timed(A, xd, (tc, tr))
                    rows.append({"workload": cfg, "scale": scale, "unaligned": unaligned, "dense_share": share, "rows": A.rows, "nnz": A.nnz,
                                 "estimated": [ec, er], "estimated_us": ms_e * 1e3, "estimated_tile_nnz": tiles_e,
                                 "tuned": [tc, tr], "tuned_us": ms_t * 1e3, "tuned_tile_nnz": tiles_t,
                                 "regret": ms_e / ms_t - 1.0})
                    log("tau family: workload %d scale %g %s share %.2f: estimate (%.2f, %.2f) %.2f us, tuned (%.2f, %.2f) %.2f us, regret %+.1f %%" % (
                        cfg, scale, "off the grid" if unaligned else "aligned", share, ec, er, ms_e * 1e3, tc, tr, ms_t * 1e3, (ms_e / ms_t - 1) * 100))
                    del A, x, xd
    return {"cases": rows, "worst_regret": max(r["regret"] for r in rows),
            "how": "regret = time of the default plan at mx_estimate_tau's fractions over that at mx_tune_tau's timed best, minus one"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", type=int, nargs="+", default=None, choices=sorted(WORKLOADS),
                    help="the first is the headline, the others go under 'others' (default: 5 2 3 4)")
    ap.add_argument("--no-sweep", action="store_true", help="tau=(0,0) only")
    ap.add_argument("--tau", type=float, nargs=2, metavar=("TAU_C", "TAU_R"), default=None,
                    help="no sweep: run this point (a profile of a fixed plan)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline (profile runs)")
    ap.add_argument("--no-unaligned", action="store_true", help="skip the variants of workloads 2 and 5 with structure off the grid")
    ap.add_argument("--all-tiles", action="store_true",
                    help="plans with MX_PLAN_ALL_TILES: every extracted chunk through the general MFMA tile kernel (profile runs)")
    ap.add_argument("--keep-tiles", action="store_true",
                    help="time the plan with MX_PLAN_KEEP_TILES instead of the default flags (profile runs of a tile form on a "
                         "matrix where a default plan drops it)")
    ap.add_argument("--scale", type=float, default=1.0,
                    help="rows of the workloads as a fraction of the benchmark's (profile runs of plans that small matrices get, "
                         "such as the one-launch form of the CSR part; the record says so and is no benchmark figure)")
    ap.add_argument("--tau-family", choices=("none", "quarter", "full"), default="quarter",
                    help="check mx_estimate_tau against mx_tune_tau over the families around workloads 2 and 5: at a quarter of "
                         "the benchmark's size (default, about half a minute), at a quarter and at full size, or not at all")
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
    t_start = time.time()
    traffic = read_traffic()
    cfgs = args.workload or [5, 2, 3, 4]

    def mode_of(cfg):
        if args.no_sweep:
            return "csr"
        return "sweep" if cfg in SWEPT else "points"
    keep = mx.MX_PLAN_ALL_TILES if args.all_tiles else None
    main_rec, (A, x) = run_workload(mx, torch, ora, cfgs[0], args.steps, args.warmup, mode_of(cfgs[0]), traffic, args.tau, keep, scale=args.scale,
                                    timed_flags=mx.MX_PLAN_KEEP_TILES if args.keep_tiles else None)
    out = {
        "metric": METRIC, "value": main_rec["gflops"], "unit": "GFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": main_rec["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": main_rec["dtype"], "data": "synthetic",
        "config": {"workload": main_rec["workload"], "rows": main_rec["rows"], "nnz": main_rec["nnz"],
                   "tau_c": main_rec["tau_c"], "tau_r": main_rec["tau_r"], "plan": main_rec["plan"],
                   "csr_variant": main_rec["csr_variant"],
                   "tau_grid": "5x5 {0,.25,.5,.75,1}^2, tau_c>=tau_r, best of sweep" if mode_of(cfgs[0]) == "sweep" and args.tau is None
                   else "no sweep: point(s) fixed"},
        "roofline": main_rec.pop("roofline"),
    }
    if not args.no_cpu:
        out["cpu_baseline"], out["cpu_all_cores"] = cpu_baseline(mx, ora, A, x)
    del A, x
    for k in ("hbm_frac_whole_spmv", "cold_cache", "rotating", "rel_l2_vs_oracle", "plan_create_ms", "plan_create_device_ms",
              "matrix_to_first_y", "plan_estimates_us", "csr_only_ms", "best_hybrid", "tile_nnz", "csr_nnz", "ms_per_step_events",
              "algorithmic_bytes", "plan_bytes_per_product", "plan_flags", "csr_one_launch", "csr_entries_kept_in_cache", "sweep", "sweep_flags", "sweep_seconds"):
        out[k] = main_rec[k]

    # what a plain device copy reaches on this GPU, next to the 8 TB/s the roofline is priced at:
    # read + written bytes over the time of back-to-back copies, at 64 MB and at 1 GiB
    copy = {}
    for label, nbytes in (("64MB", 32 << 20), ("1GiB", 1 << 29)):
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
        copy[label] = {"bytes_read_plus_written": 2 * nbytes, "GBs": 2 * nbytes / (e0.elapsed_time(e1) / reps * 1e-3) / 1e9}
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
        del src, dst
    others = {}
    for cfg in cfgs[1:]:
        r, _ = run_workload(mx, torch, ora, cfg, args.steps, args.warmup, mode_of(cfg), traffic, None, keep, scale=args.scale)
        others["workload_%d" % cfg] = r
    # the dense structure of workloads 2 and 5 off the grid of eight columns: CSR-only against the best hybrid
    if not args.no_sweep and args.tau is None and not args.no_unaligned:
        for cfg in cfgs:
            if cfg in SWEPT:
                r, _ = run_workload(mx, torch, ora, cfg, args.steps, args.warmup, "sweep", traffic, None, keep, unaligned=True, brief=True, scale=args.scale)
                others["workload_%d_unaligned" % cfg] = r
    if args.tau_family != "none" and not args.no_sweep and args.tau is None and not args.all_tiles and args.workload is None and args.scale == 1.0:
        out["tau_estimate_family"] = tau_family(mx, torch, (0.25,) if args.tau_family == "quarter" else (0.25, 1.0))
    if others:
        out["others"] = others
    out["bench_seconds"] = time.time() - t_start
    print(json.dumps(out))


if __name__ == "__main__":
    main()
