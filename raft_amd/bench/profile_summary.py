#!/usr/bin/env python3
"""Turns rocprofv3 output of bench.py into the tracked summaries under profiles/.

Run the three profiler passes on the GPU box from the repository root (TMPDIR=/tmp):

  ALL=cfg1,cfg2,cfg3_mean,cfg3_stddev,cfg3_stddev_sample,cfg4,cfg4_keys,cfg5a,cfg5b,cfg5c
  rocprofv3 --kernel-trace --stats -d OUT/kt -o kt --output-format csv -- \\
      python3 bench.py --only-kernel $ALL --steps 100 --warmup 10
  rocprofv3 --pmc FETCH_SIZE -d OUT/fetch -o fetch --output-format csv -- \\
      python3 bench.py --only-kernel $ALL --steps 6 --warmup 2 --calib-copy
  rocprofv3 --pmc WRITE_SIZE -d OUT/write -o write --output-format csv -- \\
      python3 bench.py --only-kernel $ALL --steps 6 --warmup 2 --calib-copy

  rocprofv3 --kernel-trace --stats -d OUT/ex -o ex --output-format csv -- \
      python3 bench.py --configs all --steps 40 --warmup 5 --no-cpu          (optional)

then, where git is available:  python raft_amd/bench/profile_summary.py OUT

It writes profiles/reduce_all_configs_rocprofv3.txt (per-kernel durations, raw counters, the
copy-kernel scaling, GB/s per config), profiles/row_normalize_meanvar_rocprofv3.txt when OUT/ex
exists (kernel durations of the two extra workloads of bench.py) and profiles/traffic.json (HBM bytes per launch and
kernel durations per config, with the commit they were measured at), which bench.py reads
for the `roofline.traffic` field of its report.
"""
from __future__ import annotations

import collections
import csv
import json
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent.parent
PEAK_GBPS = 8000.0
COPY_KERNEL = "__amd_rocclr_copyBuffer"
COPY_KIB = 512 * 1024  # bench.py --calib-copy moves 512 MiB per copy

# config -> (label, main kernel substring, fold kernel substring or None, input bytes, output bytes)
CONFIGS = {
    "cfg1": ("row sum fp32 10000x256", "row_wave_kernel<rmi::PolF<float, 0, 0>", None, 10240000, 40000),
    "cfg2": ("L2 row norm fp32 1000000x128 (headline)", "row_wave_kernel<rmi::PolF<float, 1, 0>", None,
             512000000, 4000000),
    "cfg3_mean": ("column mean fp32 10000000x64", "col_kernel<rmi::PolF<float, 0, 0>",
                  "fold_kernel<rmi::PolF<float, 0, 0>", 2560000000, 256),
    "cfg3_stddev": ("column stddev fp32 10000000x64 (sum of squares + epilogue)",
                    "col_kernel<rmi::PolF<float, 1, 0>", "fold_kernel<rmi::PolF<float, 1, 0>", 2560000000, 256),
    # (the sample stddev runs the same kernels as the population one, and the index-only
    # arg-max the same kernel as the key-value one: their launches are averaged together)
    "cfg3_stddev_sample": ("column stddev (sample) fp32 10000000x64", "col_kernel<rmi::PolF<float, 1, 0>",
                           "fold_kernel<rmi::PolF<float, 1, 0>", 2560000000, 256),
    "cfg4": ("row argmax fp32 65536x32000 -> {i32,f32}", "row_block_kernel<rmi::PolKvp<float, int, true>", None,
             8388608000, 524288),
    "cfg4_keys": ("matrix::argmax fp32 65536x32000 -> i32", "row_block_kernel<rmi::PolKvp<float, int, true>", None,
                  8388608000, 262144),
    "cfg5a": ("int8 4096x16384 -> int64", "row_block_kernel<rmi::PolI<signed char, 0, 0>", None, 67108864, 32768),
    "cfg5b": ("int8 16777216x8 -> int64", "row_lanes_kernel<rmi::PolI<signed char, 0, 0>", None, 134217728,
              134217728),
    "cfg5c": ("bf16 8x4194304 -> fp32 (split rows, one launch)", "row_block_kernel<rmi::PolF<rmi::bf16_t, 0, 0>",
              "fold_kernel<rmi::PolF<rmi::bf16_t, 0, 0>", 67108864, 32),
}


def _find_csv(folder: Path, suffix: str) -> Path:
    hits = sorted(folder.rglob(f"*{suffix}"))
    if not hits:
        raise SystemExit(f"no *{suffix} under {folder}")
    return hits[0]


def kernel_stats(out: Path):
    rows = list(csv.DictReader(open(_find_csv(out / "kt", "kernel_stats.csv"))))
    return {r["Name"]: r for r in rows}


def counters(out: Path, sub: str):
    rows = list(csv.DictReader(open(_find_csv(out / sub, "counter_collection.csv"))))
    agg = collections.defaultdict(list)
    for r in rows:
        agg[r["Kernel_Name"]].append(float(r["Counter_Value"]))
    return agg


def pick(d, sub):
    if sub is None:
        return None
    for k, v in d.items():
        if sub in k:
            return v
    return None


def main():
    if len(sys.argv) != 2:
        raise SystemExit(__doc__)
    out = Path(sys.argv[1])
    kt = kernel_stats(out)
    fetch, write = counters(out, "fetch"), counters(out, "write")
    copy_f, copy_w = max(pick(fetch, COPY_KERNEL)), max(pick(write, COPY_KERNEL))
    ff, wf = COPY_KIB / copy_f, COPY_KIB / copy_w
    try:
        commit = subprocess.run(["git", "-C", str(ROOT), "rev-parse", "--short", "HEAD"], capture_output=True,
                                text=True, check=True).stdout.strip()
        dirty = subprocess.run(["git", "-C", str(ROOT), "status", "--porcelain", "--", "raft_amd/csrc", "include",
                                "bench.py"], capture_output=True, text=True).stdout.strip()
        if dirty:
            commit += "+uncommitted"
    except (OSError, subprocess.CalledProcessError):
        commit = "unknown"

    lines = []
    w = lines.append
    w("rocprofv3 summary: all benchmark shapes of the dense-reduction path, one MI355X (gfx950)")
    w("=" * 87)
    w("")
    w(f"Library at commit {commit}.  Commands (run from the repository root on the GPU box, TMPDIR=/tmp):")
    w("")
    w("  ALL=cfg1,cfg2,cfg3_mean,cfg3_stddev,cfg3_stddev_sample,cfg4,cfg4_keys,cfg5a,cfg5b,cfg5c")
    w("  rocprofv3 --kernel-trace --stats -d OUT/kt -o kt --output-format csv -- \\")
    w("      python3 bench.py --only-kernel $ALL --steps 100 --warmup 10")
    w("  rocprofv3 --pmc FETCH_SIZE -d OUT/fetch -o fetch --output-format csv -- \\")
    w("      python3 bench.py --only-kernel $ALL --steps 6 --warmup 2 --calib-copy")
    w("  rocprofv3 --pmc WRITE_SIZE -d OUT/write -o write --output-format csv -- \\")
    w("      python3 bench.py --only-kernel $ALL --steps 6 --warmup 2 --calib-copy")
    w("  python raft_amd/bench/profile_summary.py OUT      (writes this file and profiles/traffic.json)")
    w("")
    w("GB/s = algorithmic bytes (input once + output once) / (kernel + fold average duration);")
    w("%peak against 8000 GB/s.  fetch / write MB = counters scaled by the copy-kernel factors.")
    w("Durations under the tracer run up to about 4 % above the same launches timed with HIP events")
    w("in bench.py on another box (tracing overhead and box-to-box spread): a kernel average here can")
    w("exceed bench.py's ms_per_step of the same workload by that much.")
    w("")
    w(f"Counter scaling from the 512 MiB device copy ({COPY_KERNEL}, {COPY_KIB} KiB read and written):")
    w(f"  FETCH_SIZE reads {copy_f:.2f} -> multiply by {ff:.4f} for KiB;  "
      f"WRITE_SIZE reads {copy_w:.2f} -> multiply by {wf:.4f} for KiB")
    w("")
    w(f"{'workload':62s} {'kernel avg us':>13s} {'fold avg us':>11s} {'alg MB':>9s} {'GB/s':>7s} {'%peak':>6s} "
      f"{'fetch MB':>10s} {'write MB':>10s}")
    doc = {"commit": commit, "peak_GBps": PEAK_GBPS,
           "source": "rocprofv3 --kernel-trace --stats / --pmc FETCH_SIZE / --pmc WRITE_SIZE on bench.py "
                     "--only-kernel, scaled by the 512 MiB copy kernel", "configs": {}}
    for name, (label, k1, k2, inb, outb) in CONFIGS.items():
        s1 = pick(kt, k1)
        if s1 is None:
            continue
        s2 = pick(kt, k2)
        t1 = float(s1["AverageNs"]) / 1e3
        t2 = float(s2["AverageNs"]) / 1e3 if s2 else 0.0
        f1, f2 = pick(fetch, k1), pick(fetch, k2) if s2 else None
        w1, w2 = pick(write, k1), pick(write, k2) if s2 else None
        avg = lambda v: sum(v) / len(v) if v else 0.0
        fe = (avg(f1) + avg(f2)) * ff * 1024
        wr = (avg(w1) + avg(w2)) * wf * 1024
        alg = inb + outb
        gbps = alg / (t1 + t2) / 1e3
        w(f"{name + '  ' + label:62s} {t1:13.2f} {t2:11.2f} {alg / 1e6:9.2f} {gbps:7.0f} {100 * gbps / PEAK_GBPS:6.1f} "
          f"{fe / 1e6:10.2f} {wr / 1e6:10.2f}")
        doc["configs"][name] = {"kernel_avg_us": t1, "fold_avg_us": t2, "algorithmic_bytes": alg,
                                "fetch_bytes": fe, "write_bytes": wr, "hbm_bytes": fe + wr,
                                "GBps": gbps, "pct_of_peak": 100 * gbps / PEAK_GBPS}
    w("")
    w("== rocprofv3 --kernel-trace --stats (durations in ns) ==")
    w(f"{'kernel':110s} {'calls':>6s} {'avg_ns':>12s} {'min_ns':>10s} {'max_ns':>10s}")
    for n, r in kt.items():
        if "rmi::" in n:
            w(f"{n[:110]:110s} {r['Calls']:>6s} {float(r['AverageNs']):12.1f} {r['MinNs']:>10s} {r['MaxNs']:>10s}")
    for agg, c in ((fetch, "FETCH_SIZE"), (write, "WRITE_SIZE")):
        w("")
        w(f"== rocprofv3 --pmc {c} (raw counter value per dispatch) ==")
        w(f"{'kernel':110s} {'disp':>5s} {'avg':>14s} {'min':>14s} {'max':>14s}")
        for k, v in agg.items():
            if "rmi::" in k or COPY_KERNEL in k:
                w(f"{k[:110]:110s} {len(v):5d} {sum(v) / len(v):14.2f} {min(v):14.2f} {max(v):14.2f}")
    (ROOT / "profiles").mkdir(exist_ok=True)
    (ROOT / "profiles" / "reduce_all_configs_rocprofv3.txt").write_text("\n".join(lines) + "\n")
    (ROOT / "profiles" / "traffic.json").write_text(json.dumps(doc, indent=1) + "\n")
    print("\n".join(lines[:40]))
    if (out / "ex").exists():
        extras(out, commit)


def extras(out: Path, commit: str):
    """Kernel durations of bench.py's extra workloads (row_normalize, meanvar, wide-row column sums)
    from OUT/ex."""
    rows = list(csv.DictReader(open(_find_csv(out / "ex", "kernel_stats.csv"))))
    kt = {r["Name"]: r for r in rows}
    lines = []
    w = lines.append
    w("rocprofv3 summary: row_normalize, meanvar, wide-row column sums, dense-slot row sums and cov, one MI355X (gfx950)")
    w("=" * 88)
    w("")
    w(f"Library at commit {commit}.  Command (run from the repository root on the GPU box, TMPDIR=/tmp):")
    w("")
    w("  rocprofv3 --kernel-trace --stats -d OUT/ex -o ex --output-format csv -- \\")
    w("      python3 bench.py --configs all --steps 40 --warmup 5 --no-cpu")
    w("")
    w("GB/s = algorithmic bytes / (kernel + fold average duration); %peak against 8000 GB/s.")
    w("")
    w(f"{'workload':50s} {'kernel':58s} {'calls':>5s} {'avg us':>8s} {'alg MB':>8s} {'GB/s':>6s} {'%peak':>6s}")
    work = [("row_normalize L2 fp32 1000000x128 (read + write)", "normalize_wave_kernel<rmi::PolF<float, 1, 0>", None,
             1024000000),
            ("row_normalize L2 fp32 1000000x129 (flat kernel)", "normalize_flat_kernel<rmi::PolF<float, 1, 0>", None,
             2 * 1000000 * 129 * 4),
            ("meanvar fp32 10000000x64 row-major (one read)", "col_kernel<rmi::PolMeanVar<float>",
             "fold_kernel<rmi::PolMeanVar<float>", 2560000512),
            ("column sum fp32 32768x4097 (whole rows)", "col_wide_kernel<rmi::PolF<float, 0, 0>",
             "fold_rows_kernel<rmi::PolF<float, 0, 0>", 32768 * 4097 * 4 + 4097 * 4),
            ("row sum fp32 2000000x66 (dense slots)", "row_dense_kernel<rmi::PolF<float, 0, 0>", None,
             2000000 * 67 * 4),
            ("L2 row norm fp32 40000000x3 (rows through LDS)", "row_small_kernel<rmi::PolF<float, 1, 0>", None,
             40000000 * 4 * 4),
            ("L2 row norm fp32 120000x1100 (one trip, 5 loads)", "row_block_kernel<rmi::PolF<float, 1, 0>", None,
             120000 * 1101 * 4),
            ("row sum fp32 525x511305 (split rows)", "row_block_kernel<rmi::PolF<float, 0, 0>",
             "fold_kernel<rmi::PolF<float, 0, 0>", 525 * 511306 * 4),
            ("stats::cov fp32 10000000x64 (data read only)", "gram_rows_kernel<float, true, true, false, true>",
             "cov_fold_kernel<float>", 2560016384),
            ("stats::cov fp32 10000000x64 (data centred in place)", "gram_rows_kernel<float, true, true, true, true>",
             "cov_fold_kernel<float>", 2 * 2560000000 + 16384)]
    for label, k1, k2, alg in work:
        s1 = pick(kt, k1)
        if s1 is None:
            continue
        s2 = pick(kt, k2)
        t1 = float(s1["AverageNs"]) / 1e3
        t2 = float(s2["AverageNs"]) / 1e3 if s2 else 0.0
        gbps = alg / (t1 + t2) / 1e3
        name1 = [n for n in kt if k1 in n][0].replace("rmi::", "").replace("void ", "")[:58]
        w(f"{label:50s} {name1:58s} {s1['Calls']:>5s} {t1:8.2f} {alg / 1e6:8.2f} {gbps:6.0f} {100 * gbps / PEAK_GBPS:6.1f}")
        if s2:
            name2 = [n for n in kt if k2 in n][0].replace("rmi::", "").replace("void ", "")[:58]
            w(f"{'':50s} {'+ ' + name2:58s} {s2['Calls']:>5s} {t2:8.2f}")
    w("")
    w("The same run's durations of the reduction kernels (ns; the caches are swept between the")
    w("single timed calls, so launch counts include those):")
    for n, r in kt.items():
        if "rmi::" in n and "normalize" not in n and "MeanVar" not in n and "col_wide" not in n \
                and "fold_rows" not in n and "row_dense" not in n and "cov::" not in n \
                and "row_small" not in n:
            w(f"  {n[:100]:100s} {r['Calls']:>6s} {float(r['AverageNs']):12.1f}")
    (ROOT / "profiles" / "row_normalize_meanvar_rocprofv3.txt").write_text("\n".join(lines) + "\n")
    print("\n".join(lines[:16]))


if __name__ == "__main__":
    main()
