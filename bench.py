#!/usr/bin/env python3
"""SpMM benchmark: GFLOPS (2*nnz*K / t) and fraction of the HBM-traffic roofline on one MI355X.

One *step* is one pass of the hot path over the benchmark's synthetic inputs:
one C = A*B for every (graph, K) workload of configurations 1-4
(citation 20k x {32,64,128}, social 233k x {32,64,128}, co-purchase 2.4M x 64,
R-MAT scale 22 x 128).  Inputs are generated on the host (seeded), copied to
HBM once, and every timed region starts with them resident.

    value        geometric mean of the per-workload GFLOPS
    ms_per_step  sum of the per-workload mean SpMM times
    roofline     social graph, K=128 (spmm_sweep_kernel is 99.6 % of its SpMM).  Its gather
                 is served by the L2s (the plan makes it so), hence "bound": "l2":
                 achieved     algorithmic bytes 4(M+1) + 8 nnz + 4 K nnz + 4 K M (the B
                              gather counted once per nonzero: every one of those rows
                              crosses the L2 -> CU path) over the time of the launches
                              of one SpMM;
                 peak         what the L2s can deliver to the CUs: 128 channels x 128 B
                              per clock x the engine clock hipDeviceProp reports
                              (l2_peak_gbs); frac = achieved / peak <= 1;
                 hbm_model_frac  the same bytes against 8 TB/s of HBM (the byte model
                              of the metric's definition; above 1, bounds nothing);
                 traffic_frac bytes the dominant kernel moves between the L2s and the
                              fabric (rocprofv3 FETCH_SIZE / WRITE_SIZE, carried in
                              MEASURED_TRAFFIC below and checked against profiles/ by
                              tests/test_bench_constants.py) over its own duration,
                              against 8 TB/s: <= 1;
                 unique_frac  the bytes that must move at least once
                              (A, every row of B once, C) over the same time.
                 Every per_workload record names its bound ("l2", "fabric",
                 "latency") and carries the same figures for the whole SpMM and
                 the per-launch times.
    cpu_baseline the FP32 CPU oracle on a bounded row sample of the same
                 social-graph workload, on this machine's host cores

Times are HIP-event times on the stream the kernels are launched on, over
exactly --steps back-to-back launches after --warmup untimed ones (the
reference's protocol: include/spmm/utils/timer_cuda.h:3-40,
spmm/mm/spmm_kernel.cu:404-424; GFLOPS formula spmm/mm/spmm_common.cpp:24-31).
"""
import argparse
import importlib
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# L2 -> CU delivery: 16 channels per XCD x 8 XCDs, 128 bytes per channel and clock
L2_BYTES_PER_CLOCK = 8 * 16 * 128
# An SpMM is timed over at least this long a region of back-to-back launches (a 4 us SpMM timed over 20
# launches is 80 us of clock ramps and launch jitter).
MIN_TIMED_MS = 10.0
SHORT_SPMM_MS = 0.05  # below this an SpMM is timed as the median of five such regions

# Run order: the microsecond-scale citation graph last.  Timed first, on a GPU that has just come
# out of idle, it was measured 25 % slower from one run to the next (clocks still ramping).
WORKLOADS = [
    ("c2_social", 32), ("c2_social", 64), ("c2_social", 128),
    ("c3_copurchase", 64),
    ("c4_rmat", 128),
    ("c1_citation", 32), ("c1_citation", 64), ("c1_citation", 128),
]
ROOFLINE_WORKLOAD = ("c2_social", 128)

# L2<->fabric bytes per launch, by kernel, of the five large workloads: rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (two runs), each scaled by what a 1 GiB copy kernel reads on the same counter (x2 for
# FETCH_SIZE, x1 for WRITE_SIZE).  Counters cannot be read from inside this process, so the figures
# are carried here, in GB as the summaries under profiles/ print them; tests/test_bench_constants.py
# fails when they differ from those files.  They are reported only for the configuration they were
# measured on: same workload, K, strategy and number of launches, scale 1, default plan.
MEASURED_TRAFFIC = {
    ("c2_social", 32): {"strategy": 6, "launches": 2, "profile": "profiles/spmm_sweep_kernel__c2_social.txt",
                        "kernels": {"spmm_sweep_kernel": 3.922, "spmm_sweep_final_kernel": 0.012}},
    ("c2_social", 64): {"strategy": 6, "launches": 2, "profile": "profiles/spmm_sweep_kernel__c2_social.txt",
                        "kernels": {"spmm_sweep_kernel": 3.998, "spmm_sweep_final_kernel": 0.010}},
    ("c2_social", 128): {"strategy": 6, "launches": 2, "profile": "profiles/spmm_sweep_kernel__c2_social.txt",
                         "kernels": {"spmm_sweep_kernel": 6.377, "spmm_sweep_final_kernel": 0.019}},
    ("c3_copurchase", 64): {"strategy": 5, "launches": 2, "profile": "profiles/spmm_ordered_kernel__c3_copurchase.txt",
                            "kernels": {"spmm_ordered_kernel": 20.428, "spmm_ordered_fixup_kernel": 0.015}},
    # (the main kernel of the routed strategy is instantiated by tile width and workgroup size, not by K)
    ("c4_rmat", 128): {"strategy": 4, "launches": 3, "profile": "profiles/spmm_routed_tiles_kernel__c4_rmat.txt",
                       "kernels": {"routed_prepare_kernel": 1.573, "spmm_routed_tiles_kernel": 32.728,
                                   "spmm_routed_final_kernel": 0.715}},
}

# What bounds each workload.
BOUND = {"c1_citation": "latency", "c2_social": "l2", "c3_copurchase": "fabric", "c4_rmat": "fabric"}
ROOF = {
    "c1_citation": "launch latency: one launch of ~2 dependent memory round trips; no bandwidth roof applies",
    "c2_social": "L2 delivery: all wavefronts walk B window by window, so every L2 holds the stretch in use; the "
                 "gather runs against the all-hit gather rate of the L2 -> CU path (l2_delivery_frac), "
                 "traffic_frac is the secondary roof",
    "c3_copurchase": "fabric: L2 misses move at the rate the L2 <-> fabric path sustains (traffic_frac)",
    "c4_rmat": "fabric: L2 misses move at the rate the L2 <-> fabric path sustains (traffic_frac)",
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def algorithmic_bytes(rows, nnz, k):
    """rowptr + (col, val) stream + B gather counted per nonzero + C write."""
    return 4 * (rows + 1) + 8 * nnz + 4 * k * nnz + 4 * k * rows


def unique_bytes(rows, cols, nnz, k):
    """Lower bound if every B row were fetched from HBM only once."""
    return 4 * (rows + 1) + 8 * nnz + 4 * k * cols + 4 * k * rows


def ensure_built():
    pkg_dir = os.path.join(ROOT, "hp-spmm-sddmm_amd")
    needed = [os.path.join(pkg_dir, "libhpspmm.so"), os.path.join(pkg_dir, "libhpspmm_graphgen.so")]
    if not all(os.path.exists(p) for p in needed):
        import __graft_entry__
        __graft_entry__.build()


def l2_delivery_ceiling(capi, graphs, dev, stream, k, steps):
    """GB/s of B-row bytes delivered to the CUs when every gather hits the L2: a matrix whose B
    (2048 rows) fits every L2, 32 M nonzeros, through the segments kernel and through the sweep kernel
    with its values bound (nothing but the gather left); the faster of the two.  Measured live, per K."""
    import torch
    g = graphs.uniform_rows(65536, 2048, 512, 99)
    B = graphs.dense_normal(g.cols, k, 99)
    d = [torch.from_numpy(a).to(dev) for a in (g.rowptr, g.col, g.val, B)]
    C = torch.empty((g.rows, k), device=dev, dtype=torch.float32)
    best = float("inf")
    for flags, bind in ((capi.PLAN_FORCE_SEGMENTS | capi.PLAN_NO_HUB_CACHE | capi.PLAN_NO_ROUTED | capi.PLAN_NO_CLUSTER, False),
                        (capi.PLAN_FORCE_SWEEP, True)):
        plan = capi.Plan(g.rows, g.cols, d[0], d[1], k, flags)
        if bind:
            plan.bind_values(d[2], stream)
        ms = capi.csr_spmm_timed(plan, d[0], d[1], d[2], d[3], C, warmup=3, iters=max(5, min(steps, 30)), stream=stream)
        plan.destroy()
        best = min(best, ms)
    return 4.0 * k * g.nnz / (best * 1e-3) / 1e9


def fabric_probe(capi, graphs, dev, stream, steps):
    """Gather rate against the size of B: the segments kernel (no hub cache, no routing) on matrices of
    512 uniformly random nonzeros per row, K = 128, with B from 1 MB (every gather an L2 hit) over sizes
    that fit the 256 MB Infinity Cache to 2 GB.  Prints one line per size: what a gather that misses the
    L2 can be served at, and whether the Infinity Cache changes that."""
    import torch
    k = 128
    for cols in (2048, 32768, 131072, 262144, 393216, 524288, 1048576, 4194304):
        g = graphs.uniform_rows(65536, cols, 512, 98)
        B = graphs.dense_normal(g.cols, k, 98)
        d = [torch.from_numpy(a).to(dev) for a in (g.rowptr, g.col, g.val, B)]
        C = torch.empty((g.rows, k), device=dev, dtype=torch.float32)
        plan = capi.Plan(g.rows, g.cols, d[0], d[1], k,
                         capi.PLAN_FORCE_SEGMENTS | capi.PLAN_NO_HUB_CACHE | capi.PLAN_NO_ROUTED | capi.PLAN_NO_CLUSTER)
        ms = capi.csr_spmm_timed(plan, d[0], d[1], d[2], d[3], C, warmup=3, iters=max(5, min(steps, 30)), stream=stream)
        plan.destroy()
        log(f"[fabric probe] B = {cols * k * 4 / 2**20:7.0f} MiB ({cols} rows of 512 B): {ms:.3f} ms, "
            f"{4.0 * k * g.nnz / (ms * 1e-3) / 1e12:.2f} TB/s of gathered rows ({g.nnz} gathers)")
        del d, C, B, g
        torch.cuda.empty_cache()


def cpu_baseline(graphs, g, B, k, C_gpu_host_rows, budget_nnz):
    """Time the CPU oracle (FP32, OpenMP, all host threads) on the first rows of the
    workload holding about budget_nnz nonzeros; also use it to check those GPU rows."""
    import numpy as np
    from oracle import oracle as o
    o.lib()
    if budget_nnz <= 0 or budget_nnz >= g.nnz:
        r_end = g.rows
    else:
        r_end = int(np.searchsorted(g.rowptr, budget_nnz, side="left"))
        r_end = max(1, min(g.rows, r_end))
    nnz_s = int(g.rowptr[r_end])
    out = np.empty((r_end, k), dtype=np.float32)
    for _ in range(2):  # warm-up / timed counts of the reference's CPU timer (timer_cpu.h:4-5)
        o.csr_spmm_f32_rows(g.rowptr, g.col, g.val, B, 0, r_end, out=out)
    reps = 2
    t0 = time.perf_counter()
    for _ in range(reps):
        o.csr_spmm_f32_rows(g.rowptr, g.col, g.val, B, 0, r_end, out=out)
    dt = (time.perf_counter() - t0) / reps
    C64, S64 = o.csr_spmm_f64_rows(g.rowptr, g.col, g.val, B, 0, min(r_end, 4096))
    err, _ = o.max_norm_err(C_gpu_host_rows[: C64.shape[0]], C64, S64)
    return {
        "value": 2.0 * nnz_s * k / dt / 1e9,
        "unit": "GFLOPS",
        "cores": o.num_threads(),
        "kind": "port",
        "sample": f"rows [0,{r_end}) of c2_social K={k}: {nnz_s} nnz, {reps} timed passes after 2 warm-ups, "
                  f"{dt * 1e3:.1f} ms per pass",
        "gpu_rows_max_normalised_err": err,
    }


# Forced strategies the plan's own choice is compared with (--strategy-table): column name, plan flags,
# the strategy the plan must end up in for the column to count.
def forced_strategies(capi):
    return [("rows", capi.PLAN_FORCE_ROWS, capi.STRATEGY_ROWS),
            ("segments", capi.PLAN_FORCE_SEGMENTS, capi.STRATEGY_SEGMENTS),
            ("ordered", capi.PLAN_CLUSTER | capi.PLAN_FORCE_SEGMENTS | capi.PLAN_NO_HUB_CACHE, capi.STRATEGY_ORDERED),
            ("routed", capi.PLAN_FORCE_ROUTED, capi.STRATEGY_ROUTED),
            ("sweep", capi.PLAN_FORCE_SWEEP, capi.STRATEGY_SWEEP)]


STRATEGY_NAMES = {1: "rows", 2: "segments", 4: "routed", 5: "ordered", 6: "sweep"}


def strategy_times(capi, g, d_rp, d_ci, d_v, d_B, d_C, k, stream, regions=2, auto_options=None):
    """Microseconds per SpMM of the default plan and of every forced strategy on one matrix: the
    smaller of `regions` timed regions of at least MIN_TIMED_MS each.  A forced strategy the plan
    could not build for this matrix (it falls back to another) reads None."""
    import torch
    out = {}
    chosen = None
    for name, flags, want in [("auto", 0, None)] + forced_strategies(capi):
        plan = capi.Plan(g.rows, g.cols, d_rp, d_ci, k, flags, options=auto_options if want is None else None)
        got = plan.info["strategy"]
        if want is None:
            chosen = got
        if want is not None and got != want:
            out[name] = None
        else:
            best = None
            for r in range(regions + 1):
                ms, _ = capi.csr_spmm_timed_min(plan, d_rp, d_ci, d_v, d_B, d_C, warmup=3 if r == 0 else 0, iters=5,
                                                min_total_ms=MIN_TIMED_MS, stream=stream)
                # (the first region after a plan has been made reads 5-10 % high: not counted)
                if r > 0:
                    best = ms if best is None else min(best, ms)
            out[name] = best * 1e3
        torch.cuda.synchronize()
        plan.destroy()
    return out, chosen


def strategy_table(capi, graphs, dev, stream, args, plan_options=None):
    """The plan's choice of strategy on generator families none of its thresholds was chosen on:
    one table line per (family, size, K) with the default plan beside every forced strategy, and
    rocSPARSE's best CSR/COO algorithm where --vendor-csv names what the host driver wrote for the
    same matrices."""
    import torch
    vendor = {}
    if args.vendor_csv:
        import re
        for line in open(args.vendor_csv):
            f = line.strip().split(",")
            if len(f) < 6 or "@" not in f[0]:
                continue
            name, sc = f[0].split("@")
            # (rocSPARSE fills the reference's cuSPARSE columns: label, ms, GFLOPS)
            ms = [float(m.group(1)) for m in re.finditer(r"cuSPARSE\([^)]*\):?\s*,([0-9.e+-]+),", line)]
            ms = [m for m in ms if m > 0]
            if ms:
                vendor[(name, float(sc), int(f[4]))] = min(ms) * 1e3
    scales = [float(x) for x in args.table_scales.split(",")]
    ks = [int(x) for x in args.table_k.split(",")]
    families = args.only.split(",") if args.only else list(graphs.HELD_OUT)
    cols = [c[0] for c in forced_strategies(capi)]
    print(f"{'family':14s} {'scale':>6s} {'rows':>9s} {'nnz':>10s} {'K':>4s} " + " ".join(f"{c:>9s}" for c in cols)
          + f" {'auto':>9s}  {'chosen':9s} {'off':>6s} {'rocSPARSE':>10s}", flush=True)
    worst = 0.0
    for name in families:
        for sc in scales:
            g = graphs.make_graph(name, sc)
            d_rp, d_ci, d_v = (torch.from_numpy(a).to(dev) for a in (g.rowptr, g.col, g.val))
            for k in ks:
                d_B = torch.from_numpy(graphs.make_dense(name, g.cols, k)).to(dev)
                d_C = torch.empty((g.rows, k), device=dev, dtype=torch.float32)
                t, chosen = strategy_times(capi, g, d_rp, d_ci, d_v, d_B, d_C, k, stream, auto_options=plan_options)
                best = min(v for c, v in t.items() if c != "auto" and v is not None)
                off = t["auto"] / best - 1
                worst = max(worst, off)
                v = vendor.get((name, sc, k))
                print(f"{name:14s} {sc:6g} {g.rows:9d} {g.nnz:10d} {k:4d} "
                      + " ".join(f"{t[c]:9.1f}" if t[c] is not None else f"{'-':>9s}" for c in cols)
                      + f" {t['auto']:9.1f}  {STRATEGY_NAMES.get(chosen, str(chosen)):9s} {100 * off:+5.1f}%"
                      + (f" {v:10.1f}" if v is not None else f" {'':>10s}"), flush=True)
                del d_B, d_C
            del d_rp, d_ci, d_v, g
            torch.cuda.empty_cache()
    print(f"largest gap between the plan's choice and the fastest forced strategy: {100 * worst:.1f} %")
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--scale", type=float, default=1.0, help="shrink every graph (debugging only; <1 is not the benchmark)")
    ap.add_argument("--only", default="", help="comma list of config names to run (debugging only)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-budget-nnz", type=int, default=0,
                    help="nonzeros in the CPU-baseline row sample (0 = the whole social graph)")
    ap.add_argument("--plan-flags", type=int, default=0)
    ap.add_argument("--plan-option", action="append", default=[], metavar="FIELD=VALUE",
                    help="a field of hpspmm_plan_options for every plan of this run (diagnostics; repeatable)")
    ap.add_argument("--no-values-bound", action="store_true",
                    help="skip the additional timing with hpspmm_plan_bind_values (keeps a profile of this "
                         "run to the launches of the figure of merit)")
    ap.add_argument("--no-launch-breakdown", action="store_true",
                    help="skip the per-launch timing and the all-hit gather probe (keeps a profile of this run "
                         "to the launches of the figure of merit)")
    ap.add_argument("--fabric-probe", action="store_true",
                    help="instead of the benchmark: the gather rate of the segments kernel against the size of B")
    ap.add_argument("--strategy-table", action="store_true",
                    help="instead of the benchmark: the default plan against every forced strategy, in microseconds, "
                         "on the families --only names (default: the generator families none of the plan's "
                         "thresholds was chosen on)")
    ap.add_argument("--table-scales", default="0.015,0.12,1.0", help="sizes for --strategy-table (for the held-out families 1 = about 10^8 nonzeros)")
    ap.add_argument("--table-k", default="32,64,128")
    ap.add_argument("--vendor-csv", default="", help="--strategy-table: a csv written by spmm_test_all --synthetic ... --csv "
                                                      "for the same matrices (name@scale), printed beside")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run three 1 GiB device-to-device copies (a kernel of known traffic, "
                         "for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py measures one GPU: this path runs on a single MI355X and no multi-GPU "
              "figure exists for it; run with --gpus 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch
    ensure_built()
    pkg = importlib.import_module("hp-spmm-sddmm_amd")
    capi, graphs = pkg.capi, pkg.graphs
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU fallback for the measured path)", file=sys.stderr)
        return 2
    capi.lib()
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream()
    plan_options = {kv.split("=", 1)[0]: int(kv.split("=", 1)[1]) for kv in args.plan_option} or None
    default_plan = args.plan_flags == 0 and plan_options is None
    clock_ghz = capi.device_info()["clock_khz"] / 1e6
    l2_peak_gbs = L2_BYTES_PER_CLOCK * clock_ghz

    if args.fabric_probe:
        fabric_probe(capi, graphs, dev, stream, args.steps)
        return 0

    if args.calibrate_copy:
        src = torch.empty(1 << 28, device=dev, dtype=torch.float32).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    # one throw-away plan first: the first call into the library loads its device image and probes the
    # workgroup -> XCD dealing once per process, which is not part of any workload's plan time
    g0 = graphs.make_graph("c0_uniform")
    w = [torch.from_numpy(a).to(dev) for a in (g0.rowptr, g0.col)]
    plan0 = capi.Plan(g0.rows, g0.cols, w[0], w[1], 32, capi.PLAN_FORCE_SEGMENTS | capi.PLAN_NO_HUB_CACHE)
    torch.cuda.synchronize()
    plan0.destroy()
    del w, g0

    if args.strategy_table:
        return strategy_table(capi, graphs, dev, stream, args, plan_options)

    workloads = WORKLOADS
    if args.only:
        keep = set(args.only.split(","))
        workloads = [w for w in WORKLOADS if w[0] in keep]
    names = []
    for n, _ in workloads:
        if n not in names:
            names.append(n)

    results = []
    cpu = None
    roofline = None
    for name in names:
        t0 = time.perf_counter()
        g = graphs.make_graph(name, args.scale)
        st = graphs.degree_stats(g.rowptr)
        log(f"[{name}] generated in {time.perf_counter() - t0:.1f}s: rows={g.rows} nnz={g.nnz} "
            f"mean_deg={st['mean_degree']:.1f} max_deg={st['max_degree']} empty={st['empty_row_fraction']:.3f} cv={st['cv']:.2f}")
        d_rp = torch.from_numpy(g.rowptr).to(dev)
        d_ci = torch.from_numpy(g.col).to(dev)
        d_v = torch.from_numpy(g.val).to(dev)
        for wname, k in workloads:
            if wname != name:
                continue
            B = graphs.make_dense(name, g.cols, k)
            d_B = torch.from_numpy(B).to(dev)
            d_C = torch.empty((g.rows, k), device=dev, dtype=torch.float32)
            # plan construction, timed twice: the first one of a kind in a process also pays for loading the
            # kernels it uses (plan_first_ms); plan_ms is what every further plan costs
            plan_times = []
            for attempt in range(2):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                plan = capi.Plan(g.rows, g.cols, d_rp, d_ci, k, args.plan_flags, options=plan_options)
                torch.cuda.synchronize()
                plan_times.append((time.perf_counter() - t0) * 1e3)
                if attempt == 0:
                    plan.destroy()
            plan_first_ms, plan_ms = plan_times
            info = plan.info
            def timed(warmup, steps):
                # hpspmm_csr_spmm_timed_min: `warmup` launches, then `steps` launches issued back to
                # back from native code between two HIP events on `stream` - the reference's timing
                # loop; when those take less than MIN_TIMED_MS, a second region of as many launches as
                # fill that time (`reps`) is what is reported.
                # (Issued one by one from Python, a 4 us SpMM is bounded by the interpreter's ~7 us
                # per call, not by the GPU.)
                torch.cuda.synchronize()
                w0 = time.perf_counter()
                ms_, reps = capi.csr_spmm_timed_min(plan, d_rp, d_ci, d_v, d_B, d_C, warmup=warmup, iters=steps,
                                                    min_total_ms=MIN_TIMED_MS, stream=stream)
                torch.cuda.synchronize()
                launches_issued = warmup + steps + (reps if reps != steps else 0)
                wall = (time.perf_counter() - w0) * 1e3 / launches_issued
                if ms_ < SHORT_SPMM_MS:
                    # an SpMM of microseconds: the median of five such regions (one region still moves
                    # by 10-15 % with whatever the clocks were doing when it began), the first one not
                    # among them: the `warmup` launches before it are a fraction of a millisecond, and
                    # the GPU has been idle while the host made the plan and the operands
                    regions = []
                    for _ in range(5):
                        m_, reps = capi.csr_spmm_timed_min(plan, d_rp, d_ci, d_v, d_B, d_C, warmup=0, iters=steps,
                                                           min_total_ms=MIN_TIMED_MS, stream=stream)
                        regions.append(m_)
                    regions.sort()
                    ms_ = regions[len(regions) // 2]
                return ms_, wall, reps

            # the figure of merit: values handed over on every call, as GESpMM receives them
            ms, wall_ms, inner_reps = timed(args.warmup, args.steps)
            # for information: values declared constant once (hpspmm_plan_bind_values), which is how
            # the reference's HP-SpMM is timed (values laid out during its preprocessing)
            ms_bound = ms
            if not args.no_values_bound:
                plan.bind_values(d_v, stream)
                ms_bound, _, _ = timed(min(args.warmup, 3), args.steps)
                plan.bind_values(None, stream)
            gflops = 2.0 * g.nnz * k / (ms * 1e-3) / 1e9
            abytes = algorithmic_bytes(g.rows, g.nnz, k)
            ubytes = unique_bytes(g.rows, g.cols, g.nnz, k)
            gbs = abytes / (ms * 1e-3) / 1e9
            # every launch of one SpMM on its own (events between the launches)
            if args.no_launch_breakdown:
                launches = [("all launches of one SpMM", ms)]
            else:
                launches = capi.csr_spmm_timed_launches(plan, d_rp, d_ci, d_v, d_B, d_C, warmup=2,
                                                        iters=max(3, min(args.steps, 50)), stream=stream)
            main_name, main_ms = max(launches, key=lambda kv: kv[1])
            rec = {
                "workload": name, "k": k, "rows": g.rows, "nnz": g.nnz, "ms": ms, "wall_ms": wall_ms,
                "inner_reps": inner_reps, "bound": BOUND.get(name, ""),
                "gflops": gflops, "ms_values_bound": ms_bound,
                "gflops_values_bound": 2.0 * g.nnz * k / (ms_bound * 1e-3) / 1e9, "algorithmic_gb": abytes / 1e9, "achieved_gbs": gbs,
                "hbm_model_frac": gbs / HBM_PEAK_GBS,
                "unique_bytes_gb": ubytes / 1e9,
                "unique_frac": ubytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                "launch_ms": {n_: t_ for n_, t_ in launches},
                "roof": ROOF.get(name, ""),
                "strategy": info["strategy"], "segment_length": info["segment_length"],
                "launches_per_spmm": info["launches_per_spmm"], "plan_ms": plan_ms, "plan_first_ms": plan_first_ms,
                "plan_over_spmm": plan_ms / ms,
                "plan_workspace_mb": info["workspace_bytes"] / 1e6,
                "plan_workspace_over_csr": info["workspace_bytes"] / (4.0 * (g.rows + 1) + 8.0 * g.nnz),
                "max_degree": st["max_degree"], "cv": st["cv"],
            }
            mt = MEASURED_TRAFFIC.get((name, k))
            if not (mt and args.scale == 1.0 and default_plan and mt["strategy"] == info["strategy"]
                    and mt["launches"] == info["launches_per_spmm"]):
                mt = None
            if mt:
                total = sum(mt["kernels"].values()) * 1e9
                rec["traffic_gb"] = total / 1e9
                rec["traffic_frac"] = total / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS
                rec["traffic_over_unique"] = total / ubytes
                rec["traffic_profile"] = mt["profile"]
            if name == "c2_social" and not args.no_launch_breakdown:
                # rows of B delivered to the CUs by the dominant kernel, against the hardware's L2 -> CU
                # rate and against what this library's own kernels reach when every gather hits the L2
                # (measured live on a 2048-row B: a ceiling of this code, not of the machine)
                gather_gbs = 4.0 * k * g.nnz / (main_ms * 1e-3) / 1e9
                ceil_gbs = l2_delivery_ceiling(capi, graphs, dev, stream, k, args.steps)
                rec["l2_peak_gbs"] = l2_peak_gbs
                rec["l2_delivery_frac"] = gather_gbs / l2_peak_gbs
                rec["l2_all_hit_measured_gbs"] = ceil_gbs
                rec["l2_delivery_over_all_hit_measured"] = gather_gbs / ceil_gbs
            results.append(rec)
            log(f"[{name} K={k}] {ms:.4f} ms  {gflops:.1f} GFLOPS  {gbs:.0f} GB/s algorithmic "
                f"({100 * gbs / HBM_PEAK_GBS:.1f}% of 8 TB/s)  strategy={info['strategy']} seg={info['segment_length']} "
                f"plan={plan_ms:.1f} ms" + ("" if args.no_values_bound else f"  [values bound: {ms_bound:.4f} ms]"))
            log("    launches: " + ", ".join(f"{n_} {t_ * 1e3:.1f} us" for n_, t_ in launches)
                + (f";  traffic {rec['traffic_gb']:.2f} GB = {rec['traffic_frac']:.2f} of 8 TB/s, "
                   f"{rec['traffic_over_unique']:.1f}x unique" if mt else "")
                + (f";  L2 delivery {rec['l2_delivery_frac']:.2f} of {l2_peak_gbs:.0f} GB/s (hardware), "
                   f"{rec['l2_delivery_over_all_hit_measured']:.2f} of {rec['l2_all_hit_measured_gbs']:.0f} GB/s "
                   f"(own all-hit run)" if "l2_delivery_frac" in rec else "")
                + (f";  timed over {inner_reps} launches" if inner_reps != args.steps else ""))
            if (name, k) == ROOFLINE_WORKLOAD:
                all_ms = sum(t_ for _, t_ in launches)  # the launches of one SpMM, each between its own events
                achieved = abytes / (all_ms * 1e-3) / 1e9
                main_traffic = mt["kernels"].get(main_name) * 1e9 if mt and main_name in mt["kernels"] else None
                roofline = {"bound": BOUND.get(name, "l2"), "achieved": achieved, "peak": l2_peak_gbs, "unit": "GB/s",
                            "frac": achieved / l2_peak_gbs,
                            "traffic": main_traffic,
                            "traffic_frac": (main_traffic / (main_ms * 1e-3) / 1e9 / HBM_PEAK_GBS) if main_traffic else None,
                            "hbm_model_frac": achieved / HBM_PEAK_GBS,
                            "unique_frac": ubytes / (all_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                            "l2_peak_gbs": l2_peak_gbs,
                            "l2_peak_source": f"{L2_BYTES_PER_CLOCK} B per clock (8 XCDs x 16 L2 channels x 128 B) x "
                                              f"{clock_ghz:.3f} GHz (hipDeviceProp clockRate)",
                            "l2_delivery_frac": rec.get("l2_delivery_frac"),
                            "l2_all_hit_measured_gbs": rec.get("l2_all_hit_measured_gbs"),
                            "l2_delivery_over_all_hit_measured": rec.get("l2_delivery_over_all_hit_measured"),
                            "kernel": f"{main_name}<{k}> (the dominant launch of one SpMM)",
                            "workload": f"{name} K={k}", "algorithmic_bytes_per_spmm": abytes,
                            "mean_launch_ms": main_ms,
                            "all_launches_ms": all_ms,
                            "whole_spmm_ms": ms,
                            "roof": ROOF.get(name, ""),
                            "note": "achieved = the algorithmic bytes of one SpMM (B gather counted once per nonzero) over "
                                    "the time of its launches; those bytes all cross the L2 -> CU path, whose hardware "
                                    "rate is the peak.  hbm_model_frac prices the same bytes against 8 TB/s of HBM, as "
                                    "the metric's byte model does: the L2s serve most of the gather, so it exceeds 1 "
                                    "and bounds nothing.  traffic / traffic_frac: measured L2<->fabric bytes of the "
                                    "dominant kernel over its own duration against 8 TB/s (<= 1); per_workload carries "
                                    "it for every large workload, where it is the figure that bounds c3 and c4."}
                if not args.no_cpu_baseline:
                    rows_chk = min(g.rows, 4096)
                    c_rows = d_C[:rows_chk].cpu().numpy()
                    t0 = time.perf_counter()
                    cpu = cpu_baseline(graphs, g, B, k, c_rows, args.cpu_budget_nnz)
                    log(f"[cpu baseline] {cpu['value']:.2f} GFLOPS on {cpu['cores']} threads "
                        f"({time.perf_counter() - t0:.1f}s); GPU rows err {cpu['gpu_rows_max_normalised_err']:.2e}")
            plan.destroy()
            del d_B, d_C, B
        del d_rp, d_ci, d_v, g
        torch.cuda.empty_cache()

    if not results:
        print("no workload selected", file=sys.stderr)
        return 2
    geo = math.exp(sum(math.log(r["gflops"]) for r in results) / len(results))
    line = {
        "metric": "SpMM GFLOPS (2*nnz*K/s), geometric mean over configs[1..4] x K, FP32 CSR, 1 MI355X",
        "value": geo,
        "unit": "GFLOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": sum(r["ms"] for r in results),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic (seeded generators, see hp-spmm-sddmm_amd/graphs.py)",
        "config": {"workload": "configs[1..4]: " + ", ".join(f"{r['workload']}/K={r['k']}" for r in results),
                   "scale": args.scale},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "value_values_bound": math.exp(sum(math.log(r["gflops_values_bound"]) for r in results) / len(results)),
        "per_workload": results,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
