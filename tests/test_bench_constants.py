"""bench.py carries measured L2<->fabric traffic per kernel as constants (hardware counters cannot
be read from inside the benchmark process).  They must be the figures of the rocprofv3 summaries
committed under profiles/: this test parses those files and fails on any drift."""
import importlib.util
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _traffic_table(path):
    """{kernel name as printed: total_GB} from the counter table of a profile summary, and
    {kernel name: avg_us} from its kernel_stats table."""
    traffic, avg_us = {}, {}
    for line in open(path):
        m = re.match(r"^(hpspmm::\S.*?)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s*$", line)
        if not m:
            continue
        # kernel_stats rows: calls avg min max pct (calls is an integer); counter rows: five decimals
        cols = line.split()
        if re.fullmatch(r"\d+", cols[-5]):
            avg_us[m.group(1)] = float(cols[-4])
        else:
            traffic[m.group(1)] = float(cols[-1])
    return traffic, avg_us


def _rows_of(names, kernel, k):
    """The rows of a table that belong to `kernel` at row length k: instantiated by K, or, for a kernel
    that is not (one instantiation in the whole file), whatever its template arguments are."""
    by_k = [n for n in names if re.match(rf"hpspmm::{kernel}<{k}[,>]", n)]
    return by_k or [n for n in names if re.match(rf"hpspmm::{kernel}<", n)]


def test_traffic_constants_match_the_profiles():
    bench = _bench()
    assert bench.MEASURED_TRAFFIC, "no measured traffic carried"
    wanted = {("c2_social", 32), ("c2_social", 64), ("c2_social", 128), ("c3_copurchase", 64), ("c4_rmat", 128)}
    assert set(bench.MEASURED_TRAFFIC) == wanted
    for (workload, k), rec in bench.MEASURED_TRAFFIC.items():
        path = os.path.join(ROOT, rec["profile"])
        assert os.path.exists(path), f"{rec['profile']} is missing"
        traffic, avg_us = _traffic_table(path)
        assert traffic, f"no counter table found in {rec['profile']}"
        assert len(rec["kernels"]) == rec["launches"]
        for kernel, gb in rec["kernels"].items():
            rows = _rows_of(traffic, kernel, k)
            assert len(rows) == 1, f"{workload} K={k}: {kernel} has {len(rows)} rows in {rec['profile']}"
            assert abs(traffic[rows[0]] - gb) <= 5e-4, \
                f"{workload} K={k} {kernel}: bench.py carries {gb} GB, {rec['profile']} says {traffic[rows[0]]} GB"
            assert _rows_of(avg_us, kernel, k), \
                f"{workload} K={k}: no duration for {kernel} in {rec['profile']}"


def test_bounded_fractions_are_bounded():
    """traffic_frac as bench.py defines it, recomputed from the profiles alone (traffic of all launches
    of one SpMM / the sum of their mean durations / 8 TB/s), is a fraction: <= 1 for every workload."""
    bench = _bench()
    for (workload, k), rec in bench.MEASURED_TRAFFIC.items():
        traffic, avg_us = _traffic_table(os.path.join(ROOT, rec["profile"]))
        total_gb = sum(rec["kernels"].values())
        total_us = sum(avg_us[_rows_of(avg_us, kernel, k)[0]] for kernel in rec["kernels"])
        frac = total_gb * 1e9 / (total_us * 1e-6) / (bench.HBM_PEAK_GBS * 1e9)
        assert 0.05 < frac <= 1.0, (workload, k, frac)


def test_l2_roofline_is_bounded():
    """The headline roofline prices the algorithmic bytes of the social graph's SpMM (B gather counted per
    nonzero) against the hardware's L2 -> CU rate: recomputed from the committed profile (kernel
    durations) and the published 2.4 GHz engine clock, it is a fraction."""
    bench = _bench()
    workload, k = bench.ROOFLINE_WORKLOAD
    rec = bench.MEASURED_TRAFFIC[(workload, k)]
    _, avg_us = _traffic_table(os.path.join(ROOT, rec["profile"]))
    total_us = sum(next(v for n, v in avg_us.items() if re.match(rf"hpspmm::{kernel}<{k}[,>]", n))
                   for kernel in rec["kernels"])
    rows, nnz = 232965, 114618680
    achieved_gbs = bench.algorithmic_bytes(rows, nnz, k) / (total_us * 1e-6) / 1e9
    peak_gbs = bench.L2_BYTES_PER_CLOCK * 2.4
    assert bench.BOUND[workload] == "l2"
    assert 0.3 < achieved_gbs / peak_gbs <= 1.0, achieved_gbs / peak_gbs
    assert achieved_gbs / bench.HBM_PEAK_GBS > 1.0  # which is why HBM is not the roof that applies
