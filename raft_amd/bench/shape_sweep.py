#!/usr/bin/env python3
"""Throughput of the reduction library over a fixed table of awkward and ordinary shapes: the
shapes the plan selector's rules were measured on (row lengths that are no power of two, rows
with tail elements, narrow and wide column reductions, 16-bit and 64-bit elements,
arg-reductions, row normalisation).  One line per shape: plan, microseconds per call, percent
of 8 TB/s (algorithmic bytes: input once + output once; row_normalize: input + output).

    python raft_amd/bench/shape_sweep.py                  # print the table
    python raft_amd/bench/shape_sweep.py --check FILE      # compare with a saved table

`--check` re-measures every shape of FILE and lists those that lost more than --points
percentage points: the guard for edits of the planner's rules (rmi_plan.hpp, rmi_launch.hpp).
Inputs rotate over at least 1 GB of buffers so that every call streams from HBM; timing is a
pair of HIP events around `--reps` back-to-back calls.
"""
from __future__ import annotations

import argparse
import ctypes as C
import re
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))


def shapes(api):
    f32, f64, bf16, i8 = api.F32, api.F64, api.BF16, api.I8
    kvp = dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, init_f=float("-inf"))
    col = dict(apply=api.ALONG_COLUMNS)
    out = []

    def rows_of(d, es, mb=512):
        return max(1, (mb << 20) // (d * es))

    # row sums
    for d in (3, 5, 9):
        out.append((f"rows f32 D={d}", f32, f32, rows_of(d, 4, 256), d, {}))
    for d in (3, 9, 17):
        out.append((f"rows bf16 D={d}", bf16, f32, rows_of(d, 2, 256), d, {}))
    for d in (5, 11):
        out.append((f"rows i8 D={d}", i8, api.I64, rows_of(d, 1, 128), d, {}))
    for d in (3, 5):
        out.append((f"rows f64 D={d}", f64, f64, rows_of(d, 8, 256), d, {}))
    out.append(("rows argmax f32 D=3", f32, api.KVP_I32_F32, rows_of(3, 4, 256), 3, kvp))
    for d in (7, 12, 16, 20, 21, 24, 32, 33, 36, 40, 41, 45, 48, 50, 54, 58, 60, 62, 64, 66, 68, 72,
              79, 83, 90, 96, 100, 125, 128, 129, 160, 200, 256, 300, 384, 768, 1000):
        out.append((f"rows f32 D={d}", f32, f32, 4_000_000 if d < 33 else 1_000_000, d, {}))
    for r, d in ((100_000, 2048), (100_000, 4096), (8192, 8192), (32768, 32768)):
        out.append((f"rows f32 {r}x{d}", f32, f32, r, d, {}))
    # rows just beyond a whole batch of the team kernel
    for d in (1025, 1100, 1500, 2049, 2500, 4097):
        out.append((f"rows f32 D={d}", f32, f32, rows_of(d, 4), d, {}))
    for d in (513, 600, 1025):
        out.append((f"rows f64 D={d}", f64, f64, rows_of(d, 8), d, {}))
    for d in (2049, 4097):
        out.append((f"rows bf16 D={d}", bf16, f32, rows_of(d, 2), d, {}))
    for d in (4097, 5000):
        out.append((f"rows i8 D={d}", i8, api.I64, rows_of(d, 1), d, {}))
    # few long rows: a last round of wide teams that would be partly filled (split rows, or
    # teams of half the width where the rows are short)
    for r, mb in ((525, 1024), (900, 1024), (1300, 1024), (1800, 1024), (525, 128), (1000, 128)):
        d = (mb << 20) // (4 * r)
        out.append((f"rows f32 {r}x{d}", f32, f32, r, d, {}))
    # long 16-bit rows of odd length (every second row starts 2 bytes off a 32-bit word)
    for d in (13593, 50337, 262145):
        out.append((f"rows bf16 D={d}", bf16, f32, rows_of(d, 2), d, {}))
    for d in (9, 17, 25, 33, 35, 63, 65, 67, 129):
        out.append((f"rows f64 D={d}", f64, f64, 2_000_000, d, {}))
    for d in (33, 36, 65, 66, 76, 100, 129, 130, 132, 250, 260, 513):
        out.append((f"rows bf16 D={d}", bf16, f32, 2_000_000, d, {}))
    for d in (17, 33, 47, 70, 90, 150, 270, 500):
        out.append((f"rows i8 D={d}", i8, api.I64, rows_of(d, 1, 256), d, {}))
    for d in (20, 33, 62, 66, 129):
        out.append((f"rows argmax f32 D={d}", f32, api.KVP_I32_F32, 4_000_000 if d < 33 else 1_000_000, d, kvp))
    # column sums, 512 MB each
    for d in (1, 2, 3, 5, 7, 12, 16, 20, 33, 48, 63, 64, 65, 100, 128, 129, 200, 256, 260, 300):
        out.append((f"cols f32 D={d}", f32, f32, rows_of(d, 4), d, col))
    for d in (3, 8, 9, 17, 33, 65, 100, 127, 128, 300):
        out.append((f"cols bf16 D={d}", bf16, f32, rows_of(d, 2), d, col))
    for d in (17, 33, 50, 65, 127):
        out.append((f"cols i8 D={d}", i8, api.I64, rows_of(d, 1), d, col))
    for d in (3, 33, 100):
        out.append((f"cols f64 D={d}", f64, f64, rows_of(d, 8), d, col))
    for d in (516, 600, 768, 1000, 1100, 1400, 1536, 2049, 2300, 3000, 3500, 4096, 4097, 5000, 5120,
              8191, 11000, 20000, 50000):
        out.append((f"cols wide f32 D={d}", f32, f32, rows_of(d, 4), d, col))
    for d in (260, 640, 1025, 2560, 4097):
        out.append((f"cols wide f64 D={d}", f64, f64, rows_of(d, 8), d, col))
    for d in (1030, 3000, 6000, 16400):
        out.append((f"cols wide bf16 D={d}", bf16, f32, rows_of(d, 2), d, col))
    for d in (129, 2049, 4097, 10000):
        out.append((f"cols argmax f32 D={d}", f32, api.KVP_I32_F32, rows_of(d, 4), d, dict(col, **kvp)))
    for d in (4100, 8200, 20000):
        out.append((f"cols i8 D={d}", i8, api.I64, rows_of(d, 1), d, col))
    # row normalisation (L2), 512 MB in + 512 MB out
    for d in (5, 8, 16, 20, 32, 33, 50, 64, 100, 128, 129, 200, 220, 250, 256, 300, 401, 500, 512, 777, 1000,
              1024, 4096, 10000):
        out.append((f"normalize f32 D={d}", f32, f32, rows_of(d, 4), d, "normalize"))
    for d in (3, 5, 9, 33, 100, 128, 130, 256, 1000, 4096):
        out.append((f"normalize bf16 D={d}", bf16, bf16, rows_of(d, 2), d, "normalize"))
    out.append(("normalize f32 D=3", f32, f32, rows_of(3, 4), 3, "normalize"))
    out.append(("normalize f32 D=1100", f32, f32, rows_of(1100, 4), 1100, "normalize"))
    out.append(("normalize bf16 D=2049", bf16, bf16, rows_of(2049, 2), 2049, "normalize"))
    for d in (25, 33, 65, 128, 250):
        out.append((f"normalize f64 D={d}", f64, f64, rows_of(d, 8), d, "normalize"))
    return out


def measure(api, lib, torch, case, reps):
    name, in_dt, out_dt, rows, cols, kw = case
    tdt = {api.F32: torch.float32, api.F64: torch.float64, api.BF16: torch.bfloat16,
           api.I8: torch.int8}[in_dt]
    es = api.DTYPE_SIZE[in_dt]
    n = rows * cols
    nbuf = max(2, min(8, -(-(1 << 30) // (n * es))))
    if in_dt == api.I8:
        bufs = [torch.randint(-128, 128, (n,), device="cuda", dtype=torch.int8) for _ in range(nbuf)]
    else:
        bufs = [torch.randn(n, device="cuda", dtype=torch.float32).to(tdt) for _ in range(nbuf)]
    sptr = torch.cuda.current_stream().cuda_stream
    if kw == "normalize":
        d = api.make_desc(in_dt, in_dt, rows, cols, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
        outs = [torch.empty_like(b) for b in bufs]
        plan = "normalize"
        nbytes = 2 * n * es

        def call(i):
            return lib.rmi_row_normalize(C.byref(d), bufs[i % nbuf].data_ptr(),
                                         outs[i % nbuf].data_ptr(), 1e-8, sptr)
    else:
        d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
        n_out = rows if d.apply == api.ALONG_ROWS else cols
        out = torch.empty(n_out * api.DTYPE_SIZE[out_dt], dtype=torch.uint8, device="cuda")
        nws = lib.rmi_reduce_workspace_bytes(C.byref(d))
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device="cuda")
        pl = api.plan_query(d)
        plan = f"{api.PLAN_NAME[pl.kind]}/{pl.passes}"
        nbytes = n * es + n_out * api.DTYPE_SIZE[out_dt]

        def call(i):
            return lib.rmi_reduce(C.byref(d), bufs[i % nbuf].data_ptr(), out.data_ptr(),
                                  ws.data_ptr(), nws, sptr)
    for i in range(3):
        rc = call(i)
        assert rc == 0, (name, api.status_string(rc))
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(4):  # the fastest of four rounds: single rounds are now and then 10-20 % slow
        e0.record()
        for i in range(reps):
            call(i)
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) / reps * 1e3)
    pct = nbytes / (best * 1e-6) / 8e12 * 100.0
    del bufs
    torch.cuda.empty_cache()
    return plan, best, pct


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reps", type=int, default=10)
    ap.add_argument("--filter", default="", help="substring of the shape names to run")
    ap.add_argument("--check", default=None, help="saved table to compare with")
    ap.add_argument("--points", type=float, default=4.0, help="loss that counts as a regression")
    args = ap.parse_args()
    import torch

    from raft_amd import _capi as api
    lib = api.load()
    saved = {}
    if args.check:
        for line in open(args.check):
            m = re.match(r"^(.+?)\s{2,}(\S+)\s+([\d.]+) us\s+([\d.]+) %$", line.rstrip())
            if m:
                saved[m.group(1)] = float(m.group(4))
    worse = []
    print(f"{'shape':28s}  {'plan':14s} {'per call':>10s}  {'of 8 TB/s':>9s}")
    for case in shapes(api):
        if args.filter not in case[0]:
            continue
        if saved and case[0] not in saved:
            continue
        plan, us, pct = measure(api, lib, torch, case, args.reps)
        note = ""
        if case[0] in saved:
            note = f"   (saved {saved[case[0]]:.1f} %)"
            if pct < saved[case[0]] - args.points:
                worse.append((case[0], saved[case[0]], pct))
                note += "  REGRESSION"
        print(f"{case[0]:28s}  {plan:14s} {us:8.1f} us  {pct:7.1f} %{note}", flush=True)
    if args.check:
        print(f"\n{len(worse)} shapes lost more than {args.points} points")
        sys.exit(1 if worse else 0)


if __name__ == "__main__":
    main()
