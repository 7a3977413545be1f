#!/usr/bin/env python3
"""Benchmark of the CSR hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config {1,2,3,4,5}]

A step is one pass of the hot path over one batch of synthetic input resident in
HBM: one SpMV (configs 1-3), one SpMM (config 4) or one CG iteration (config 5; a
run is exactly `steps` iterations).  The default workload is config 2, the one the
headline metric is quoted on.  Prints ONE JSON line.

Protocol (benchmarks/spmv/main.cpp:52-62 of the reference): device-resident inputs,
warm-up calls, then K calls; the K calls are timed as one region bracketed by device
synchronisation, and the dominant kernel is timed per launch with HIP events
attached to its dispatches in that same region.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# roofline.traffic is not measured inside this run (hardware counters need rocprofv3 around the process)
TRAFFIC_SOURCE = ("profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run of this kernel, "
                  "scaled by a copy kernel of known size; null when this run's kernel time is more than 20 % off "
                  "the time recorded with the reading")


def traffic_from_profiles(kernel_key, kernel_ms):
    """HBM bytes per launch measured with rocprofv3 --pmc (profiles/traffic.json), or None.

    The figure belongs to the kernel as it was when it was profiled: it is given only when this run's
    mean kernel time is within 20 % of the time recorded beside it, otherwise None (stale or unprofiled)."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        entry = json.load(f).get(kernel_key)
    if not entry or not entry.get("kernel_ms_at_profile"):
        return None
    if abs(kernel_ms - entry["kernel_ms_at_profile"]) > 0.2 * entry["kernel_ms_at_profile"]:
        return None
    return entry["hbm_bytes_per_launch"]


def calibrate_gather(full=False):
    """Rates of the two things a column-blocked SpMV launch spends its time on, measured with the library's
    calibration kernel (lapis_hip_calibrate_gather): streaming the matrix, and gathering x from L2 one
    128-byte line per request.  On this chip the two do not overlap: the times ADD.  With `full` the whole
    table (merge factors 1..16, the three cache levels) is returned as well."""
    import torch
    from lapis_amd import hip
    gathers = 1 << 26
    # 1 GiB: 12 bytes per gather fit; the full table has modes in which only half of the wavefronts stream,
    # each from a region of its own
    stream = torch.zeros(1 << (28 if full else 27), dtype=torch.float64, device="cuda")
    x = torch.zeros(1 << 23, dtype=torch.float64, device="cuda")       # 64 MB window at most
    sink = torch.zeros(4096, dtype=torch.float64, device="cuda")
    l2 = 1 << 20
    only_stream = hip.calibrate_gather(None, 0, 0, stream, gathers, sink)
    only_gather = hip.calibrate_gather(x, l2, 1, None, gathers, sink)
    both = hip.calibrate_gather(x, l2, 1, stream, gathers, sink)
    stream_rate = only_stream["stream_bytes"] / (only_stream["ms"] * 1e-3)  # bytes/s
    line_rate = only_gather["gathers"] / (only_gather["ms"] * 1e-3)          # 128-byte lines/s
    out = {"stream_only_ms": only_stream["ms"], "stream_TB_per_s": stream_rate / 1e12,
           "gather_only_ms": only_gather["ms"], "gather_lines_G_per_s": line_rate / 1e9,
           "both_ms": both["ms"], "sum_of_parts_ms": only_stream["ms"] + only_gather["ms"],
           "window": "1 MB of x (L2 resident)", "gathers": only_gather["gathers"],
           "stream_bytes": only_stream["stream_bytes"]}
    if full:
        table = []
        for window, label in ((16 << 10, "16 KB (vector cache)"), (l2, "1 MB (L2)"), (64 << 20, "64 MB (HBM)")):
            for lanes in (1, 2, 4, 8, 16):
                for with_stream in (False, True):
                    if window != l2 and lanes != 1:
                        continue
                    r = hip.calibrate_gather(x, window, lanes, stream if with_stream else None, gathers, sink)
                    lines = r["gathers"] / lanes
                    table.append({"window": label, "lanes_per_line": lanes, "stream": with_stream, "ms": r["ms"],
                                  "gather_lines_G_per_s": lines / (r["ms"] * 1e-3) / 1e9,
                                  "predicted_ms": (r["stream_bytes"] / stream_rate + lines / line_rate) * 1e3
                                  if window == l2 else None})
        out["table"] = table
        out["modes"] = calibrate_modes(hip, x, l2, stream, sink, stream_rate, line_rate)
    del stream, x, sink
    return out


def calibrate_modes(hip, x, window, stream, sink, stream_rate, line_rate):
    """The same stream and the same gathers in other arrangements (lapis_hip_calibrate_mix): does any of them let
    a compute unit overlap the two?  805 MB of stream and 42.4 M single-line gathers from an L2-resident window --
    what config 2 sends after the column-blocked copy has merged its gathers -- unless a row says otherwise."""
    import torch
    cu_count = torch.zeros(16 * 256, dtype=torch.int32, device="cuda")
    S, G = 12 << 26, 42.4e6
    both = lambda **kw: dict(kw)
    rows = [
        ("stream only", both(threads=512, stream_in_flight=3, stream_policy=1), S, 0),
        ("stream only, 16 wavefronts, 12 loads in flight", both(threads=1024, stream_in_flight=12, stream_policy=1), S, 0),
        ("stream only, on 64 compute units", both(threads=1024, workgroups=64, stream_in_flight=12, stream_policy=1), S, 0),
        ("gathers only", both(threads=512, gathers_in_flight=4), 0, G),
        ("gathers only, 16 wavefronts, 8 in flight", both(threads=1024, gathers_in_flight=8), 0, G),
        ("every wavefront does both, 8 per CU", both(threads=512, stream_in_flight=3, gathers_in_flight=2, stream_policy=1), S, G),
        ("every wavefront does both, 16 per CU", both(threads=1024, stream_in_flight=6, gathers_in_flight=4, stream_policy=1), S, G),
        ("every wavefront does both, 2 workgroups of 8 per CU", both(threads=512, workgroups=512, stream_in_flight=6, gathers_in_flight=4, stream_policy=1), S, G),
        ("both, next step's stream issued behind the gathers", both(threads=1024, stream_in_flight=6, gathers_in_flight=4, stream_policy=1, stream_behind=1), S, G),
        ("roles by wavefront: 4 stream, 12 gather", both(threads=1024, stream_in_flight=6, gathers_in_flight=4, stream_policy=1, roles=1, producers=4), S, G),
        ("roles by wavefront: 4 stream (12 in flight), 8 gather", both(threads=768, stream_in_flight=12, gathers_in_flight=4, stream_policy=1, roles=1, producers=4), S, G),
        ("roles by wavefront: 8 stream, 8 gather", both(threads=1024, stream_in_flight=6, gathers_in_flight=4, stream_policy=1, roles=1, producers=8), S, G),
        ("roles by wavefront: 3 stream, 5 gather", both(threads=512, stream_in_flight=12, gathers_in_flight=4, stream_policy=1, roles=1, producers=3), S, G),
        ("roles by workgroup: 2 x 8 wavefronts per CU", both(threads=512, workgroups=512, stream_in_flight=6, gathers_in_flight=4, stream_policy=1, roles=2), S, G),
        ("roles by workgroup: 2 x 4 wavefronts per CU", both(threads=256, workgroups=512, stream_in_flight=12, gathers_in_flight=4, stream_policy=1, roles=2), S, G),
        ("both, stream loads sc0 sc1", both(threads=1024, stream_in_flight=6, gathers_in_flight=4, stream_policy=2), S, G),
        ("both, stream loads sc0 sc1 nt", both(threads=1024, stream_in_flight=6, gathers_in_flight=4, stream_policy=3), S, G),
        ("both, stream straight to LDS", both(threads=1024, stream_in_flight=6, gathers_in_flight=4, stream_policy=4), S, G),
        ("roles by wavefront, stream straight to LDS", both(threads=768, stream_in_flight=12, gathers_in_flight=4, stream_policy=4, roles=1, producers=4), S, G),
        ("stream kept in L2, alone", both(threads=512, stream_in_flight=3, stream_in_l2=1), S, 0),
        ("stream kept in L2 + gathers (a perfect prefetch)", both(threads=512, stream_in_flight=3, gathers_in_flight=2, stream_in_l2=1), S, G),
        ("stream alone through the scalar cache (64-byte loads)", both(threads=1024, workgroups=512, stream_in_flight=3, scalar=1), S // 4, 0),
        ("both + helper wavefronts touching the stream through the scalar cache, every 128 B", both(threads=512, stream_in_flight=3, gathers_in_flight=4, scalar=2, scalar_ahead=4, scalar_stride=128), S, G),
        ("both + helper wavefronts touching the stream through the scalar cache, every 64 B", both(threads=512, stream_in_flight=3, gathers_in_flight=4, scalar=2, scalar_ahead=4, scalar_stride=64), S, G),
        ("stream + such helpers, no gathers", both(threads=512, stream_in_flight=3, scalar=2, scalar_ahead=4, scalar_stride=128), S, 0),
    ]
    out = []
    for label, mode, sbytes, gathers in rows:
        r = hip.calibrate_mix(mode, x, window, stream, sbytes, gathers, cu_count, sink)
        lines = r["gathers"]
        out.append({"mode": label, "ms": r["ms"], "stream_MB": r["stream_bytes"] / 1e6, "gather_lines_M": lines / 1e6,
                    "stream_TB_per_s": r["stream_bytes"] / (r["ms"] * 1e-3) / 1e12,
                    "gather_lines_G_per_s": lines / (r["ms"] * 1e-3) / 1e9,
                    "sum_of_parts_ms": (r["stream_bytes"] / stream_rate + lines / line_rate) * 1e3,
                    "cus_with_both_roles": r["cus_with_both_roles"], **mode})
    return out


def colgroup_request_floor(stats, A, cal, value_bytes):
    """Floor of the workgroup column-blocked kernel from the calibrated rates: the matrix copy streamed once
    plus one L2 request per distinct 128-byte line of x a tile touches.  A block of R rows puts
    d = R * mean_row_len * (128 / value_bytes) / ncols entries into every line of x on average; with columns
    drawn uniformly a wave instruction's 64 column-sorted neighbours merge into (1 - exp(-d)) / d requests per
    entry.  Returned only for matrices without long rows (those go to blocks of their own)."""
    import math
    if stats["max_row_len"] >= max(2048.0, 16.0 * stats["mean_row_len"]):
        return None
    rows = 16384 if A.nrows > 8192 else (8192 if A.nrows > 4096 else 4096)
    d = rows * stats["mean_row_len"] * (128.0 / value_bytes) / max(1, A.ncols)
    per_entry = (1.0 - math.exp(-d)) / d if d > 1e-9 else 1.0
    lines = A.nnz * per_entry
    copy_bytes = A.nnz * (4 + value_bytes)
    floor_ms = (copy_bytes / (cal["stream_TB_per_s"] * 1e12) + lines / (cal["gather_lines_G_per_s"] * 1e9)) * 1e3
    return {"entries_per_line": d, "requests_per_entry": per_entry, "gather_lines_per_launch": lines,
            "streamed_bytes_per_launch": copy_bytes, "floor_ms": floor_ms}


def cpu_baseline_spmv(A, x, budget_s=12.0):
    """The OpenMP restatement of the reference loop nest, timed on this host's cores."""
    from oracle.oracle import Oracle
    omp = Oracle(omp=True)
    y = np.zeros(A.nrows, dtype=A.val.dtype)
    omp.spmv(A.pos, A.crd, A.val, x, y, parallel=True)  # warm-up, first touch
    t0 = time.perf_counter()
    omp.spmv(A.pos, A.crd, A.val, x, y, parallel=True)
    one = time.perf_counter() - t0
    reps = int(min(2000, max(3, budget_s / max(one, 1e-6))))
    t0 = time.perf_counter()
    for _ in range(reps):
        omp.spmv(A.pos, A.crd, A.val, x, y, parallel=True)
    dt = (time.perf_counter() - t0) / reps
    return {"value": A.spmv_bytes() / dt / 1e9, "unit": "GB/s", "cores": omp.max_threads(), "kind": "port",
            "sample": "%d calls of the full workload (%d rows, %d non-zeros), OpenMP static row split, "
                      "%.3f ms per call; Kokkos is not installed, so this is the C restatement of the "
                      "reference loop nest" % (reps, A.nrows, A.nnz, dt * 1e3),
            "gflops": 2.0 * A.nnz / dt / 1e9}


def run_spmv(args, cfg):
    import torch
    from lapis_amd import generators as gen
    from lapis_amd import hip
    if args.workload:
        maker0, t_mi300a, t_h100 = gen.PUBLISHED[args.workload]
        published = {"matrix": args.workload, "MI300A_s": t_mi300a, "H100_s": t_h100,
                     "source": "benchmarks/plots/spmv.csv of the reference (mean of 1000 fenced calls)"}
        cfg = 0
    else:
        published = None
    name, maker, dtype = {
        0: ("%s (structure of the reference's published matrix), SpMV fp64" % args.workload,
            (lambda: (maker0(), None)) if args.workload else None, np.float64),
        1: ("config1: SpMV fp64, 2-D 5-point Laplacian 256x256", gen.config1, np.float64),
        2: ("config2: SpMV fp64, n=4194304, Poisson(16) rows, uniform random sorted columns, int32 indices",
            gen.config2, np.float64),
        3: ("config3: SpMV fp32, n=2097152, power-law rows (exponent 2, min 1, cap 200000, mean 30)", gen.config3,
            np.float32),
    }[cfg]
    t0 = time.perf_counter()
    A, x = maker()
    if x is None:
        x = gen.uniform_vector(A.ncols, 77)
    log("generated %s: %d rows, %d nnz in %.1f s" % (name, A.nrows, A.nnz, time.perf_counter() - t0))
    dev = lambda a: torch.from_numpy(a).cuda()
    pos, crd, val, dx = dev(A.pos), dev(A.crd), dev(A.val), dev(x)
    y = torch.zeros(A.nrows, dtype=torch.float64 if dtype == np.float64 else torch.float32, device="cuda")
    t0 = time.perf_counter()
    plan = hip.CsrPlan(A.nrows, A.ncols, pos, crd, value_bytes=np.dtype(dtype).itemsize)
    torch.cuda.synchronize()
    plan_ms = (time.perf_counter() - t0) * 1e3
    build_ms = None
    csr_ms = None
    if args.kernel == "colblock":
        t0 = time.perf_counter()
        plan.build_colblock(crd, val, layout=args.colblock_layout)
        torch.cuda.synchronize()
        build_ms = (time.perf_counter() - t0) * 1e3
    elif args.kernel:
        plan.set_kernel({"subwarp": 1, "rowblock": 2, "nnzsplit": 3}[args.kernel], args.width)
    else:
        # The library decides (lapis_hip_csr_plan_analyze): it builds the column-blocked copy where the
        # row/column statistics call for it.  The CSR kernel the plan would otherwise launch is timed first,
        # so that the number of calls after which the copy has paid for itself can be stated.
        for _ in range(3):
            hip.spmv(plan, A.nrows, A.ncols, pos, crd, val, dx, y)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(10):
            hip.spmv(plan, A.nrows, A.ncols, pos, crd, val, dx, y)
        torch.cuda.synchronize()
        csr_ms = (time.perf_counter() - t0) / 10 * 1e3
        y.zero_()
        before = plan.stats()["kernel_name"]
        t0 = time.perf_counter()
        plan.analyze(crd, val)
        torch.cuda.synchronize()
        if plan.stats()["kernel_name"] != before:
            build_ms = (time.perf_counter() - t0) * 1e3
    stats = plan.stats()
    for _ in range(args.warmup):
        hip.spmv(plan, A.nrows, A.ncols, pos, crd, val, dx, y)
    torch.cuda.synchronize()
    hip.kernel_timing_start(args.steps)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        hip.spmv(plan, A.nrows, A.ncols, pos, crd, val, dx, y)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    kt = hip.kernel_timing_stop()
    bytes_step = A.spmv_bytes()
    ms = elapsed / args.steps * 1e3
    update_ms = None
    if stats["kernel_name"] == "colblock":
        # what new values of the same structure cost: one gather pass through the kept permutation
        plan.update_values(val)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(5):
            plan.update_values(val)
        torch.cuda.synchronize()
        update_ms = (time.perf_counter() - t0) / 5 * 1e3
    # The same set-up a second time: the first plan of a process also pays for loading the kernels
    # and for the first large allocations.
    plan_ms_again = build_ms_again = None
    if build_ms is not None and not args.kernel:
        t0 = time.perf_counter()
        plan2 = hip.CsrPlan(A.nrows, A.ncols, pos, crd, value_bytes=np.dtype(dtype).itemsize)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        plan2.analyze(crd, val)
        torch.cuda.synchronize()
        plan_ms_again, build_ms_again = (t1 - t0) * 1e3, (time.perf_counter() - t1) * 1e3
        del plan2
    family = "colgroup" if stats["colblock_layout_name"] == "group" else stats["kernel_name"]
    kernel_name = "%s<%s>" % (plan.kernel_name(), "double" if dtype == np.float64 else "float")
    achieved = bytes_step / (kt["mean_ms"] * 1e-3) / 1e9
    out = {
        "metric": "CSR SpMV %s achieved HBM GB/s" % ("fp64" if dtype == np.float64 else "fp32"),
        "value": bytes_step / (ms * 1e-3) / 1e9, "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f64" if dtype == np.float64 else "f32", "data": "synthetic",
        "config": {"workload": name, "nrows": A.nrows, "nnz": A.nnz, "seed": {0: 77, 1: 1001, 2: 2002, 3: 3003}[cfg],
                   "colblock_build_ms": build_ms, "mean_chunk_col_span": stats["mean_chunk_col_span"],
                   "algorithmic_bytes_per_step": bytes_step, "kernel": stats["kernel_name"],
                   "colblock_layout": stats["colblock_layout_name"],
                   "width": stats["width"], "chunk": stats["chunk"],
                   "reference_vector_length": stats["reference_vector_length"], "plan_ms": plan_ms,
                   "csr_kernel_ms_per_call": csr_ms, "colblock_update_values_ms": update_ms,
                   # calls of this matrix after which building the copy (outside the timed region) has paid back
                   "break_even_calls": (build_ms / (csr_ms - ms) if build_ms and csr_ms and csr_ms > ms else None),
                   # a second plan of the same matrix in the same process
                   "plan_ms_second_plan": plan_ms_again, "colblock_build_ms_second_plan": build_ms_again,
                   "break_even_calls_second_plan": (build_ms_again / (csr_ms - ms)
                                                    if build_ms_again and csr_ms and csr_ms > ms else None)},
        "pct_of_hbm_peak": 100.0 * bytes_step / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "gflops": 2.0 * A.nnz / (ms * 1e-3) / 1e9,
        "roofline": {"bound": "hbm", "kernel": kernel_name, "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": traffic_from_profiles("%s_config%d" % (plan.kernel_name()[5:-7], cfg), kt["mean_ms"]) if cfg else None,
                     "traffic_source": TRAFFIC_SOURCE,
                     "kernel_ms_mean": kt["mean_ms"], "kernel_ms_median": kt["median_ms"],
                     "kernel_ms_min": kt["min_ms"], "launches_timed": kt["count"]},
    }
    if family == "colgroup" and not args.no_calibration:
        cal = calibrate_gather(full=args.calibrate_gather)
        floor = colgroup_request_floor(stats, A, cal, np.dtype(dtype).itemsize)
        out["calibration"] = cal
        if floor:
            # what bounds this kernel is not HBM: its traffic is 1.35 x algorithmic at 3.7 TB/s.  It is the
            # requests its compute units can keep in flight; see calibrate_gather().
            # It is the floor of THIS kernel shape (every wavefront streams and gathers), not of the chip:
            # the graded figure is roofline.frac.
            out["roofline"]["secondary"] = dict(floor, bound="line_requests_in_flight", achieved_ms=kt["mean_ms"],
                                                fraction_of_scheme_floor=floor["floor_ms"] / kt["mean_ms"],
                                                model="stream_bytes / stream rate + gather lines / line rate, both "
                                                      "calibrated in this run with wavefronts that do both; "
                                                      "wavefronts with one role each overlap the two by about a "
                                                      "fifth in the calibration kernel (bench.py --calibrate-gather)")
    if args.graph or cfg == 1:
        # Launch-bound sizes: the same calls captured once into a HIP graph (10 per graph) and
        # replayed, which takes the Python and launch overhead of each call out of the loop.
        per_graph = 10
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for _ in range(per_graph):
                    hip.spmv(plan, A.nrows, A.ncols, pos, crd, val, dx, y)
        torch.cuda.synchronize()
        replays = max(1, args.steps // per_graph)
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(replays):
            graph.replay()
        torch.cuda.synchronize()
        gms = (time.perf_counter() - t0) / (replays * per_graph) * 1e3
        out["graph_replay"] = {"calls_per_graph": per_graph, "ms_per_step": gms,
                               "GB/s": bytes_step / (gms * 1e-3) / 1e9}
    if args.host_buffers:
        # The generated-module entry takes HOST arrays (the reference's Python path):
        # every call uploads the matrix and vectors and copies y back.  Reported beside
        # `value`, never as it.
        from lapis_amd.module import LAPISModule
        mod = LAPISModule()
        spec = ((A.nrows, A.ncols), (A.nrows + 1, A.nnz, A.nnz))
        yh = np.zeros(A.nrows, dtype=dtype)
        mod.spmv(A.pos, A.crd, A.val, spec, x, yh)  # warm-up
        reps = 3
        t0 = time.perf_counter()
        for _ in range(reps):
            mod.spmv(A.pos, A.crd, A.val, spec, x, yh)
        hms = (time.perf_counter() - t0) / reps * 1e3
        out["host_buffers"] = {"entry": "py_spmv via LAPISModule.spmv (host arrays, H2D + kernel + D2H per call)",
                               "ms_per_call": hms, "GB/s": bytes_step / (hms * 1e-3) / 1e9}
        if dtype == np.float64:
            # the opt-in resident path of the same module: matrix bound once, vectors as dual views
            t0 = time.perf_counter()
            Ad = mod.bind_csr(A.pos, A.crd, A.val, spec)
            bind_ms = (time.perf_counter() - t0) * 1e3
            t0 = time.perf_counter()
            for _ in range(reps):
                Ad.spmv(x, yh)
            mixed_ms = (time.perf_counter() - t0) / reps * 1e3
            xv, yv = mod.dual_view(x.copy()), mod.dual_view(np.zeros(A.nrows))
            Ad.spmv(xv, yv)
            yv.sync_host()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                Ad.spmv(xv, yv)
            yv.sync_host()
            rms = (time.perf_counter() - t0) / args.steps * 1e3
            out["host_buffers"]["resident"] = {
                "entry": "LAPISModule.bind_csr(...).spmv: matrix, plan and column-blocked copy kept on the device",
                "bind_ms": bind_ms, "ms_per_call_numpy_vectors": mixed_ms,
                "ms_per_call_dual_views": rms, "GB/s_dual_views": bytes_step / (rms * 1e-3) / 1e9,
                "ratio_to_c_abi": rms / ms}
            Ad.release()
    if published:
        # fenced per-call protocol of the published numbers: one call, one synchronise
        t0 = time.perf_counter()
        for _ in range(args.steps):
            hip.spmv(plan, A.nrows, A.ncols, pos, crd, val, dx, y)
            torch.cuda.synchronize()
        fenced = (time.perf_counter() - t0) / args.steps
        published["this_run_fenced_s"] = fenced
        published["speedup_vs_MI300A"] = published["MI300A_s"] / fenced
        published["speedup_vs_H100"] = published["H100_s"] / fenced
        out["published_comparison"] = published
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_spmv(A, x)
    return out


def run_spmm(args):
    import torch
    from lapis_amd import generators as gen
    from lapis_amd import hip
    k = args.k
    if args.workload:
        # structure of one of the reference's published SpMV matrices (fp64 in the table), here as the
        # sparse operand of an fp32 SpMM: a matrix WITH column locality, beside config 4 which has none
        A = gen.PUBLISHED[args.workload][0]()
        A = gen.CSR(A.nrows, A.ncols, A.pos, A.crd, A.val.astype(np.float32))
        B = gen.uniform_matrix(A.ncols, k, 4005).astype(np.float32)
        name = "%s (structure of the reference's published matrix) as fp32 SpMM operand, B %dx%d row-major" % (
            args.workload, A.ncols, k)
    else:
        A, B = gen.config4()
        if k != B.shape[1]:
            B = gen.uniform_matrix(A.ncols, k, 4005).astype(np.float32)
        name = "config4: SpMM fp32, A 1048576^2 with 32 nnz/row, B 1048576x%d row-major" % k
        if args.spmm_fold_b:
            # the same matrix with its columns folded onto the first R rows of B: what the kernel would cost if B
            # were that much smaller (the most that blocking B could buy)
            R = args.spmm_fold_b
            crd = (A.crd % R).astype(np.int32)
            rows = np.repeat(np.arange(A.nrows, dtype=np.int64), np.diff(A.pos))
            order = np.lexsort((crd, rows))
            A = gen.CSR(A.nrows, R, A.pos, crd[order], A.val[order])
            B = np.ascontiguousarray(B[:R])
            name = "config4 with the columns of A folded onto %d rows of B (%d x %d fp32, %.1f MB)" % (
                R, R, k, R * k * 4 / 1e6)
    dev = lambda a: torch.from_numpy(a).cuda()
    pos, crd, val, dB = dev(A.pos), dev(A.crd), dev(A.val), dev(B)
    C = torch.zeros(A.nrows, k, dtype=torch.float32, device="cuda")
    if args.spmm_kernel != "auto":
        os.environ["LAPIS_HIP_SPMM_KERNEL"] = args.spmm_kernel
    plan = hip.CsrPlan(A.nrows, A.ncols, pos, crd, value_bytes=4)  # its band statistics pick the kernel
    stats = plan.stats()
    for _ in range(args.warmup):
        hip.spmm(A.nrows, A.ncols, pos, crd, val, dB, C, plan=plan)
    torch.cuda.synchronize()
    hip.kernel_timing_start(args.steps)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        hip.spmm(A.nrows, A.ncols, pos, crd, val, dB, C, plan=plan)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    kt = hip.kernel_timing_stop()
    # A streamed once, B counted once, C written once (the read of C for the accumulate is not counted)
    bytes_step = 8 * A.nnz + 4 * (A.nrows + 1) + 4 * A.ncols * k + 4 * A.nrows * k
    ms = elapsed / args.steps * 1e3
    achieved = bytes_step / (kt["mean_ms"] * 1e-3) / 1e9
    out = {
        "metric": "CSR x dense SpMM fp32 achieved HBM GB/s", "value": bytes_step / (ms * 1e-3) / 1e9, "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": name, "nrows": A.nrows, "nnz": A.nnz, "k": k, "seed": 4004,
                   "algorithmic_bytes_per_step": bytes_step, "spmm_kernel": args.spmm_kernel,
                   "near_diagonal_fraction": stats["near_diagonal_fraction"], "mean_row_len": stats["mean_row_len"]},
        "pct_of_hbm_peak": 100.0 * bytes_step / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "gflops": 2.0 * A.nnz * k / (ms * 1e-3) / 1e9,
        "roofline": {"bound": "hbm", "kernel": "%s<float>" % hip.spmm_last_kernel(), "achieved": achieved,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": traffic_from_profiles("spmm_config4", kt["mean_ms"])
                     if not args.workload and k == 64 and not args.spmm_fold_b else None,
                     "traffic_source": TRAFFIC_SOURCE,
                     "kernel_ms_mean": kt["mean_ms"], "kernel_ms_median": kt["median_ms"],
                     "kernel_ms_min": kt["min_ms"], "launches_timed": kt["count"]},
    }
    if not args.no_cpu:
        from oracle.oracle import Oracle
        omp = Oracle(omp=True)
        rows = A.nrows // 8  # bounded sample: the first eighth of the rows
        sub_pos = A.pos[:rows + 1]
        Cc = np.zeros((rows, k), np.float32)
        t0 = time.perf_counter()
        omp.spmm(sub_pos, A.crd, A.val, B, Cc, parallel=True)
        dt = time.perf_counter() - t0
        frac = rows / A.nrows
        out["cpu_baseline"] = {"value": bytes_step * frac / dt / 1e9, "unit": "GB/s", "cores": omp.max_threads(),
                               "kind": "port", "sample": "first %d of %d rows, one call, %.1f ms" % (rows, A.nrows, dt * 1e3)}
    return out


def run_cg(args):
    import torch
    from lapis_amd import generators as gen
    from lapis_amd import hip
    A, b = gen.config5()
    n = A.nrows
    dev = lambda a: torch.from_numpy(a).cuda()
    pos, crd, val, db = dev(A.pos), dev(A.crd), dev(A.val), dev(b)
    x = torch.empty(n, dtype=torch.float64, device="cuda")
    work = torch.empty(4 * n, dtype=torch.float64, device="cuda")
    plan = hip.CsrPlan(n, n, pos, crd)
    t0 = time.perf_counter()
    plan.analyze(crd, val)  # the library's decision, as lapis_hip_pcg_f64_i32 makes it for solves of 64+ iterations
    torch.cuda.synchronize()
    analyze_ms = (time.perf_counter() - t0) * 1e3
    hip.pcg(plan, n, pos, crd, val, db, None, 0.0, max(1, args.warmup), x, work=work)
    torch.cuda.synchronize()
    hip.kernel_timing_start(args.steps)
    t0 = time.perf_counter()
    iters, relres = hip.pcg(plan, n, pos, crd, val, db, None, 0.0, args.steps, x, work=work)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    kt = hip.kernel_timing_stop()
    assert iters == args.steps
    spmv_bytes = A.spmv_bytes()
    bytes_step = spmv_bytes + 2 * 2 * 8 * n + 3 * 3 * 8 * n  # SpMV + 2 dots + 3 axpy
    ms = elapsed / args.steps * 1e3
    achieved = spmv_bytes / (kt["mean_ms"] * 1e-3) / 1e9
    out = {
        "metric": "CG fp64 achieved HBM GB/s per iteration", "value": bytes_step / (ms * 1e-3) / 1e9, "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f64", "data": "synthetic",
        "config": {"workload": "config5: unpreconditioned CG fp64, 7-point Laplacian 192^3, %d iterations" % args.steps,
                   "nrows": n, "nnz": A.nnz, "seed": 5005, "algorithmic_bytes_per_step": bytes_step,
                   "final_relres": relres, "plan_analyze_ms": analyze_ms},
        "pct_of_hbm_peak": 100.0 * bytes_step / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "gflops": (2.0 * A.nnz + 2 * 2 * n + 3 * 3 * n) / (ms * 1e-3) / 1e9,
        "roofline": {"bound": "hbm", "kernel": "%s<double>" % plan.kernel_name(),
                     "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": traffic_from_profiles("cg_spmv_config5", kt["mean_ms"]),
                     "traffic_source": TRAFFIC_SOURCE,
                     "kernel_ms_mean": kt["mean_ms"], "kernel_ms_median": kt["median_ms"],
                     "launches_timed": kt["count"]},
    }
    if not args.no_cpu:
        from oracle.oracle import Oracle
        omp = Oracle(omp=True)
        p, Ap = b.copy(), np.zeros(n)
        reps = 3
        t0 = time.perf_counter()
        for _ in range(reps):  # one iteration's kernels: SpMV + 2 dots + 3 axpy
            Ap[:] = 0
            omp.spmv(A.pos, A.crd, A.val, p, Ap, parallel=True)
            omp.dot(p, Ap, parallel=True)
            omp.dot(Ap, Ap, parallel=True)
            omp.axpby(1.0, p, 0.5, Ap, p, parallel=True)
            omp.axpby(1.0, Ap, 0.5, p, Ap, parallel=True)
            omp.axpby(1.0, p, 0.5, Ap, p, parallel=True)
        dt = (time.perf_counter() - t0) / reps
        out["cpu_baseline"] = {"value": bytes_step / dt / 1e9, "unit": "GB/s", "cores": omp.max_threads(), "kind": "port",
                               "sample": "%d iterations' worth of SpMV + 2 dots + 3 axpy on the full workload" % reps}
    if args.module:
        # the same solve through the generated-module boundary: py_pcg copies every operand per call, the
        # resident handles keep the matrix and the vectors on the device
        from lapis_amd.module import LAPISModule
        del pos, crd, val, db, x, work
        torch.cuda.empty_cache()
        mod = LAPISModule()
        spec = ((n, n), (n + 1, A.nnz, A.nnz))
        t0 = time.perf_counter()
        _, it, _ = mod.pcg(A.pos, A.crd, A.val, spec, b, np.ones(n), 0.0, args.steps)
        per_call = time.perf_counter() - t0
        Ad = mod.bind_csr(A.pos, A.crd, A.val, spec)
        bv, xv = mod.dual_view(b), mod.dual_view(np.zeros(n))
        Ad.pcg(bv, None, 0.0, 2, xv)
        t0 = time.perf_counter()
        _, it2, _ = Ad.pcg(bv, None, 0.0, args.steps, xv)
        resident = time.perf_counter() - t0
        out["through_module"] = {
            "py_pcg_ms_per_call": per_call * 1e3, "py_pcg_iterations": int(it),
            "py_pcg_note": "host operands copied in and out by the call, Jacobi preconditioner of ones",
            "resident_ms_per_iteration": resident / args.steps * 1e3, "resident_iterations": int(it2),
            "resident_GB_per_s": bytes_step / (resident / args.steps) / 1e9}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--config", type=int, default=2, choices=[1, 2, 3, 4, 5])
    ap.add_argument("--workload", choices=["Laplace3D_100", "Elasticity3D_60"], default=None,
                    help="SpMV on the structure of one of the reference's published matrices instead of a config")
    ap.add_argument("--kernel", choices=["subwarp", "rowblock", "nnzsplit", "colblock"], default=None,
                    help="force an SpMV kernel family instead of the plan's choice")
    ap.add_argument("--colblock-layout", choices=["auto", "wave", "group"], default="auto",
                    help="layout of the column-blocked copy (auto = group)")
    ap.add_argument("--width", type=int, default=0, help="lanes per row with --kernel subwarp (0 = the reference's rule)")
    ap.add_argument("--k", type=int, default=64, help="columns of B for the SpMM workloads (config 4)")
    ap.add_argument("--spmm-fold-b", type=int, default=0,
                    help="config 4 with the column indices of A taken modulo this many rows of B (an experiment: "
                         "what a smaller B would cost)")
    ap.add_argument("--spmm-kernel", choices=["auto", "wave", "group", "lds"], default="auto",
                    help="SpMM kernel: the plan's choice, the wavefront-per-row kernel, or the LDS-staged row-block kernel")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--graph", action="store_true",
                    help="also time the calls replayed from a HIP graph (always done for config 1)")
    ap.add_argument("--host-buffers", action="store_true",
                    help="also time the generated-module entry point, which takes host arrays (PCIe-inclusive)")
    ap.add_argument("--calibrate-gather", action="store_true",
                    help="print the whole gather/stream calibration table (merge factors, cache levels) instead of "
                         "the three rows the secondary roofline needs")
    ap.add_argument("--no-calibration", action="store_true", help="skip the gather/stream calibration launches")
    ap.add_argument("--module", action="store_true",
                    help="config 5: also run the solve through the generated-module boundary (py_pcg with host "
                         "operands, and the device-resident handles)")
    ap.add_argument("--no-others", action="store_true",
                    help="with the default configuration: do not also run configurations 3, 4 and 5 (the 'others' block)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch the library's copy kernel on 1 GiB three times, the known-size reference "
                         "that rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if args.workload and args.config != 4:
        args.config = 1  # takes the SpMV path; run_spmv swaps the matrix in
    if args.steps is None:
        args.steps = {1: 1000, 2: 200, 3: 200, 4: 20, 5: 100}[args.config]
    if args.warmup is None:
        args.warmup = {1: 10, 2: 10, 3: 10, 4: 2, 5: 2}[args.config]
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU: the HIP library has no CPU path")
    if args.calibrate_copy:
        from lapis_amd import hip
        src = torch.ones(1 << 27, dtype=torch.float64, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            hip.copy(src, dst)
        torch.cuda.synchronize()
        del src, dst
    if args.config in (1, 2, 3):
        out = run_spmv(args, args.config)
    elif args.config == 4:
        out = run_spmm(args)
    else:
        out = run_cg(args)
    if args.config == 2 and not args.workload and not args.no_others and not args.calibrate_gather:
        out["others"] = run_others(args)
    print(json.dumps(out), flush=True)


def run_others(args):
    """The other configurations beside the headline, each for at most 20 steps, without CPU legs: what the
    same library does on the power-law SpMV (3), the SpMM (4) and CG (5).  Keys per configuration:
    ms_per_step, kernel, kernel_ms_mean, frac (of the 8 TB/s roofline, for the dominant kernel),
    algorithmic_bytes_per_step, GB/s (whole step)."""
    import copy
    import gc
    import torch
    others = {}
    for cfg, runner in ((3, lambda a: run_spmv(a, 3)), (4, run_spmm), (5, run_cg)):
        a = copy.copy(args)
        a.config, a.no_cpu, a.no_calibration, a.graph, a.host_buffers = cfg, True, True, False, False
        a.kernel, a.workload, a.k, a.spmm_kernel = None, None, 64, "auto"
        a.spmm_fold_b, a.module = 0, False
        a.steps, a.warmup = min(20, {3: 20, 4: 20, 5: 20}[cfg]), 2
        gc.collect()
        torch.cuda.empty_cache()
        try:
            r = runner(a)
        except Exception as e:  # the headline line must not be lost to a failure here
            others["config%d" % cfg] = {"error": repr(e)}
            continue
        others["config%d" % cfg] = {
            "workload": r["config"]["workload"], "metric": r["metric"], "steps": r["steps"],
            "ms_per_step": r["ms_per_step"], "GB/s": r["value"], "kernel": r["roofline"]["kernel"],
            "kernel_ms_mean": r["roofline"]["kernel_ms_mean"], "frac": r["roofline"]["frac"],
            "algorithmic_bytes_per_step": r["config"]["algorithmic_bytes_per_step"], "dtype": r["dtype"],
            "pct_of_hbm_peak_whole_step": r["pct_of_hbm_peak"]}
    return others


if __name__ == "__main__":
    main()
