#!/usr/bin/env python3
"""Benchmark of the dense-reduction path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs all|headline]

A "step" is one reduction call (one pass of the hot path over one matrix).  The
headline workload is the L2 row norm of a row-major fp32 1,000,000 x 128 matrix
(N(0,1), sqrt fused); the other benchmark shapes are timed the same way and
reported under "configs".  Inputs are generated on the device from fixed seeds and
are resident in HBM before timing starts; consecutive steps read different
buffers whose total size is at least twice the 256 MB Infinity Cache, so every step
streams from HBM.  Timing uses HIP events recorded on the stream the kernels run on.
Per config, beside the back-to-back average: the same launches replayed from a HIP
graph, the same buffer every step (cache-resident where it fits), and single calls
timed one by one after a 768 MB scratch sweep has evicted the caches (median and
minimum of the repetitions; the method of the reference's benchmark fixture,
cpp/bench/prims/common/benchmark.hpp:138-155).

Prints one JSON line; `roofline.by_config` holds ms per step, algorithmic bytes and the
fraction of 8 TB/s for every workload (the long per-workload records go to
bench_details.json).  `roofline.achieved` = algorithmic bytes (input read once +
output written once) / average launch duration.  `roofline.traffic` is NOT measured in
this run: it is read from profiles/traffic.json, which raft_amd/bench/profile_summary.py
writes from rocprofv3 counter runs of this same program (the file names the commit it
was measured at).  `cpu_baseline` times the OpenMP host implementation of the same
semantics (oracle/, kind "port") on this machine's cores.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_HBM_GBPS = 8000.0  # MI355X published HBM3E bandwidth


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--configs", default="all",
                    help="all | headline | comma list of cfg names (cfg1,cfg2,cfg3_mean,...)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-check", action="store_true", help="skip the correctness gate")
    ap.add_argument("--only-kernel", default=None,
                    help="run just this config's launches (for rocprofv3), no JSON extras")
    ap.add_argument("--calib-copy", action="store_true",
                    help="with --only-kernel: also run 5 device copies of 512 MiB, the known-size "
                         "kernel that rocprofv3 byte counters are scaled against")
    return ap.parse_args()


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the reduction path shards by rows "
              "with no exchange; no multi-GPU figure is produced). Use --gpus 1.",
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from raft_amd import _capi as api
    from raft_amd import device as dev

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    lib = api.load()
    torch.cuda.set_device(0)
    devc = torch.device("cuda:0")
    stream = torch.cuda.current_stream()
    sptr = stream.cuda_stream

    # Inputs come from a counter-based generator (raft_amd/bench/synth.py): element i of a
    # buffer is a function of (seed, i) alone, so the host can recompute any of them; the
    # seeds are echoed in the output line.
    from raft_amd.bench import synth

    def mk_normal(rows, cols, seed, mean=0.0, std=1.0):
        return synth.normal_device(seed, rows * cols, mean, std, devc)

    def mk_uniform(rows, cols, seed):
        return synth.uniform_device(seed, rows * cols, devc)

    def mk_int8(rows, cols, seed):
        return synth.int8_device(seed, rows * cols, devc)

    def mk_bf16(rows, cols, seed):
        return mk_uniform(rows, cols, seed).to(torch.bfloat16)

    def mk_logits_with_ties(rows, cols, seed):
        # rows whose hash is 0 mod 100 (1 % of them) get their maximum copied to one to three
        # further columns, all drawn from the same counter-based stream
        x = mk_normal(rows, cols, seed).view(rows, cols)
        h = torch.from_numpy(synth.bits_host(seed + 1000, np.arange(rows * 4)).view(np.int64)
                             .reshape(rows, 4)).to(devc)
        lsr = lambda z, k: (z >> k) & ((1 << (64 - k)) - 1)  # noqa: E731
        tie_rows = torch.nonzero(lsr(h[:, 0], 8) % 100 == 0).view(-1)
        mx = x[tie_rows].amax(dim=1)
        for j in range(3):  # 1..3 further copies of the row maximum
            hj = h[tie_rows, j + 1]
            pos = lsr(hj, 20) % cols
            keep = torch.ones_like(pos, dtype=torch.bool) if j == 0 else (hj & 1) == 1
            x[tie_rows[keep], pos[keep]] = mx[keep]
        return x.view(-1)

    f32 = np.float32
    WORK = {
        # name: (description, maker, rows, cols, desc kwargs, out dtype bytes)
        "cfg1": dict(desc="row sum fp32 10000x256 U[-1,1) seed 0", make=lambda s: mk_uniform(10000, 256, s),
                     seed=0, rows=10000, cols=256, in_dt=api.F32, out_dt=api.F32, kw={}),
        "cfg2": dict(desc="L2 row norm (sqrt) fp32 1000000x128 N(0,1)", make=lambda s: mk_normal(1000000, 128, s),
                     seed=2, rows=1000000, cols=128, in_dt=api.F32, out_dt=api.F32,
                     kw=dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)),
        "cfg3_mean": dict(desc="column mean fp32 10000000x64 N(3,2)", make=lambda s: mk_normal(10000000, 64, s, 3.0, 2.0),
                          seed=3, rows=10000000, cols=64, in_dt=api.F32, out_dt=api.F32,
                          kw=dict(apply=api.ALONG_COLUMNS, final_op=api.FIN_MUL_CONST,
                                  final_scalar=float(f32(1.0) / f32(10000000)))),
        "cfg3_stddev": dict(desc="column stddev fp32 10000000x64 N(3,2)", make=lambda s: mk_normal(10000000, 64, s, 3.0, 2.0),
                            seed=3, rows=10000000, cols=64, in_dt=api.F32, out_dt=api.F32,
                            kw=dict(apply=api.ALONG_COLUMNS, main_op=api.MAIN_SQ,
                                    final_op=api.FIN_STDDEV_FROM_SUMSQ,
                                    final_scalar=float(f32(1.0) / f32(10000000)), final_scalar2=1.0),
                            needs_mean=True),
        "cfg3_stddev_sample": dict(desc="column stddev (sample) fp32 10000000x64 N(3,2)",
                                   make=lambda s: mk_normal(10000000, 64, s, 3.0, 2.0),
                                   seed=3, rows=10000000, cols=64, in_dt=api.F32, out_dt=api.F32,
                                   kw=dict(apply=api.ALONG_COLUMNS, main_op=api.MAIN_SQ,
                                           final_op=api.FIN_STDDEV_FROM_SUMSQ,
                                           final_scalar=float(f32(1.0) / f32(9999999)),
                                           final_scalar2=float(f32(f32(1.0) / f32(9999999)) * f32(10000000))),
                                   needs_mean=True),
        "cfg4": dict(desc="row argmax (KVP int32,fp32) fp32 65536x32000 N(0,1), ties in 1% of rows",
                     make=lambda s: mk_logits_with_ties(65536, 32000, s), seed=4, rows=65536, cols=32000,
                     in_dt=api.F32, out_dt=api.KVP_I32_F32,
                     kw=dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, init_i=0,
                             init_f=float("-inf"))),
        "cfg4_keys": dict(desc="matrix::argmax (int32 index only) fp32 65536x32000 N(0,1), ties in 1% of rows",
                          make=lambda s: mk_logits_with_ties(65536, 32000, s), seed=4, rows=65536, cols=32000,
                          in_dt=api.F32, out_dt=api.I32,
                          kw=dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, final_op=api.FIN_KEY,
                                  init_i=0, init_f=float("-inf"))),
        "cfg5a": dict(desc="row sum int8->int64 4096x16384", make=lambda s: mk_int8(4096, 16384, s),
                      seed=5, rows=4096, cols=16384, in_dt=api.I8, out_dt=api.I64, kw={}),
        "cfg5b": dict(desc="row sum int8->int64 16777216x8", make=lambda s: mk_int8(16777216, 8, s),
                      seed=6, rows=16777216, cols=8, in_dt=api.I8, out_dt=api.I64, kw={}),
        "cfg5c": dict(desc="row sum bf16->fp32 8x4194304 (split rows, last workgroup of a row folds)",
                      make=lambda s: mk_bf16(8, 4194304, s), seed=7, rows=8, cols=4194304,
                      in_dt=api.BF16, out_dt=api.F32, kw={}),
    }
    HEADLINE = "cfg2"

    if args.configs == "all":
        names = list(WORK)
    elif args.configs == "headline":
        names = [HEADLINE]
    else:
        names = [n for n in args.configs.split(",") if n]
    if args.only_kernel:
        names = args.only_kernel.split(",")
    if HEADLINE not in names and not args.only_kernel:
        names.insert(0, HEADLINE)

    def n_out(w):
        return w["rows"] if w["kw"].get("apply", api.ALONG_ROWS) == api.ALONG_ROWS else w["cols"]

    def alg_bytes(w):
        return (w["rows"] * w["cols"] * api.DTYPE_SIZE[w["in_dt"]]
                + n_out(w) * api.DTYPE_SIZE[w["out_dt"]])

    TORCH_OUT = {api.F32: torch.float32, api.I64: torch.int64, api.I32: torch.int32}

    # > 512 MB written between single timed calls: evicts the 256 MB memory-side cache
    flush_buf = torch.empty(768 << 20, dtype=torch.uint8, device=devc)

    def run_config(name, steps, warmup, check=True, extras=True):
        w = WORK[name]
        in_bytes = w["rows"] * w["cols"] * api.DTYPE_SIZE[w["in_dt"]]
        # enough distinct inputs that a buffer is long out of the 256 MB Infinity Cache when
        # its turn comes again: at least 512 MB in rotation (cfg1: 53 buffers of 10 MB)
        nbuf = max(2, min(64, -(-(512 << 20) // in_bytes)))
        bufs = [w["make"](w["seed"] + 7919 * i) for i in range(nbuf)]
        no = n_out(w)
        out_bytes = no * api.DTYPE_SIZE[w["out_dt"]]
        outs = [torch.zeros(out_bytes, dtype=torch.uint8, device=devc) for _ in range(nbuf)]
        kw = dict(w["kw"])
        descs = []
        aux = []
        for i in range(nbuf):
            # the workspace below is zero-filled once and then only used by the library
            d = api.make_desc(w["in_dt"], w["out_dt"], w["rows"], w["cols"],
                              flags=api.FLAG_WORKSPACE_ZEROED, **kw)
            if w.get("needs_mean"):
                m = bufs[i].view(w["rows"], w["cols"]).mean(dim=0, dtype=torch.float64).to(torch.float32)
                aux.append(m)
                d.final_aux = m.data_ptr()
            descs.append(d)
        plan = api.plan_query(descs[0])
        ws_bytes = lib.rmi_reduce_workspace_bytes(C.byref(descs[0]))
        ws = torch.zeros(max(ws_bytes, 16), dtype=torch.uint8, device=devc)
        wsp = ws.data_ptr()
        in_ptrs = [b.data_ptr() for b in bufs]
        out_ptrs = [o.data_ptr() for o in outs]
        refs = [C.byref(d) for d in descs]
        call = lib.rmi_reduce

        def step(i):
            j = i % nbuf
            rc = call(refs[j], in_ptrs[j], out_ptrs[j], wsp, ws_bytes, sptr)
            if rc != 0:
                raise RuntimeError(f"{name}: rmi_reduce -> {api.status_string(rc)}")

        for i in range(warmup):
            step(i)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(stream)
        for i in range(steps):
            step(i)
        e1.record(stream)
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        ev_ms = e0.elapsed_time(e1)
        ms = ev_ms / steps
        res = dict(workload=w["desc"], plan=api.PLAN_NAME[plan.kind], passes=plan.passes,
                   grid_blocks=plan.grid_blocks, buffers=nbuf, ms_per_step=ms,
                   wall_ms_per_step=wall_ms / steps,
                   alg_bytes=alg_bytes(w), GBps=alg_bytes(w) / (ms * 1e-3) / 1e9,
                   rows_per_s=w["rows"] / (ms * 1e-3))
        res["pct_of_peak"] = 100.0 * res["GBps"] / PEAK_HBM_GBPS
        res["hbm_traffic_bytes_profile"] = PROFILE_TRAFFIC.get(name)
        if not extras:  # profiler runs: the timed launches only
            return res, bufs, outs

        # the same launches replayed from a HIP graph: removes host launch gaps, which
        # dominate the shapes whose kernel is only a few microseconds long
        try:
            gsteps = max(nbuf, min(steps, 64))
            side = torch.cuda.Stream()
            side.wait_stream(stream)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                gptr = side.cuda_stream
                with torch.cuda.graph(graph, stream=side):
                    for i in range(gsteps):
                        j = i % nbuf
                        rc = call(refs[j], in_ptrs[j], out_ptrs[j], wsp, ws_bytes, gptr)
                        assert rc == 0
            stream.wait_stream(side)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            reps = max(1, steps // gsteps)
            e0.record(stream)
            for _ in range(reps):
                graph.replay()
            e1.record(stream)
            torch.cuda.synchronize()
            gms = e0.elapsed_time(e1) / (reps * gsteps)
            res["graph_ms_per_step"] = gms
            res["graph_GBps"] = alg_bytes(w) / (gms * 1e-3) / 1e9
            del graph
        except Exception as ex:  # noqa: BLE001
            res["graph_error"] = str(ex)[:200]

        # same buffer every step (cache-resident when the input fits the Infinity Cache)
        if in_bytes <= (256 << 20):
            for i in range(5):
                call(refs[0], in_ptrs[0], out_ptrs[0], wsp, ws_bytes, sptr)
            torch.cuda.synchronize()
            e0.record(stream)
            for i in range(steps):
                call(refs[0], in_ptrs[0], out_ptrs[0], wsp, ws_bytes, sptr)
            e1.record(stream)
            torch.cuda.synchronize()
            cms = e0.elapsed_time(e1) / steps
            res["same_buffer_ms_per_step"] = cms
            res["same_buffer_GBps"] = alg_bytes(w) / (cms * 1e-3) / 1e9

        # single calls, caches evicted before each: median and minimum of the repetitions
        # (a pair of events around one call carries a few microseconds of its own)
        reps = 20
        times = []
        for i in range(reps):
            flush_buf.fill_(i & 0xFF)
            e0.record(stream)
            step(i)
            e1.record(stream)
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1))
        times.sort()
        res["flushed_single_call_us"] = {"median": times[reps // 2] * 1e3, "min": times[0] * 1e3,
                                         "reps": reps}

        if check:
            res["check"] = check_config(name, w, bufs[0], outs[0], aux[0] if aux else None)
        return res, bufs, outs

    # ------------------------------------------------------------------
    # correctness gate: oracle on a bounded sample + full-size properties
    # ------------------------------------------------------------------
    def check_config(name, w, buf, out_raw, aux):
        from tests import _util as u
        rows, cols = w["rows"], w["cols"]
        info = {}
        kw = dict(w["kw"])
        if w["out_dt"] == api.I32 and kw.get("final_op") == api.FIN_KEY:
            keys = out_raw.view(torch.int32).to(torch.int64)
            x = buf.view(rows, cols)
            ok = True
            ar = torch.arange(cols, device=devc, dtype=torch.int64)
            for r0 in range(0, rows, 4096):
                blk = x[r0:r0 + 4096]
                eq = blk == blk.amax(dim=1)[:, None]
                first = torch.where(eq, ar[None, :], torch.full((), cols, device=devc, dtype=torch.int64)).amin(dim=1)
                ok &= bool(torch.equal(first, keys[r0:r0 + 4096]))
            info["full_size_first_max_property"] = ok
            ns = 256
            sample = x[:ns].contiguous().cpu().numpy().reshape(-1)
            d = api.make_desc(w["in_dt"], w["out_dt"], ns, cols, **kw)
            ek, _ = u.oracle_reduce(d, sample)
            info["oracle_sample_rows"] = ns
            info["oracle_exact"] = bool(np.array_equal(keys[:ns].cpu().numpy(), ek))
            info["pass"] = ok and info["oracle_exact"]
            return info
        if w["out_dt"] == api.KVP_I32_F32:
            kv = out_raw.view(torch.int32).view(rows, 2)
            keys = kv[:, 0].to(torch.int64)
            vals = kv[:, 1].contiguous().view(torch.float32)
            x = buf.view(rows, cols)
            ok = True
            for r0 in range(0, rows, 4096):
                blk = x[r0:r0 + 4096]
                mx = blk.amax(dim=1)
                eq = blk == mx[:, None]
                ar = torch.arange(cols, device=devc, dtype=torch.int64)
                first = torch.where(eq, ar[None, :], torch.full((), cols, device=devc, dtype=torch.int64)).amin(dim=1)
                ok &= bool(torch.equal(first, keys[r0:r0 + 4096]))
                ok &= bool(torch.equal(mx, vals[r0:r0 + 4096]))
            info["full_size_first_max_property"] = ok
            ns = 256
            sample = buf.view(rows, cols)[:ns].contiguous().cpu().numpy().reshape(-1)
            d = api.make_desc(w["in_dt"], w["out_dt"], ns, cols, **kw)
            ek, ev = u.oracle_reduce(d, sample)
            gk = keys[:ns].cpu().numpy()
            gv = vals[:ns].cpu().numpy().astype(np.float64)
            info["oracle_sample_rows"] = ns
            info["oracle_exact"] = bool(np.array_equal(gk, ek) and np.array_equal(gv, ev))
            info["pass"] = ok and info["oracle_exact"]
            return info
        along_rows = kw.get("apply", api.ALONG_ROWS) == api.ALONG_ROWS
        if along_rows:
            ns = min(rows, max(1, (32 << 20) // (cols * api.DTYPE_SIZE[w["in_dt"]])))
            tsample = buf.view(rows, cols)[:ns].contiguous()
            sample = (tsample.view(torch.int16).cpu().numpy().view(np.uint16) if w["in_dt"] == api.BF16
                      else tsample.cpu().numpy()).reshape(-1)
            d = api.make_desc(w["in_dt"], w["out_dt"], ns, cols, **kw)
            exp = u.oracle_reduce(d, sample)
            got = out_raw.view(TORCH_OUT[w["out_dt"]])[:ns].cpu().numpy()
            info["oracle_sample_rows"] = ns
            if w["out_dt"] == api.I64:
                info["oracle_exact"] = bool(np.array_equal(got, exp))
                # full size: total of all row sums against an independent device reduction
                tot = int(out_raw.view(torch.int64).sum().item())
                ref = int(buf.view(-1).to(torch.int64).sum().item()) if buf.numel() <= (1 << 28) else \
                    sum(int(c.to(torch.int64).sum().item()) for c in buf.view(-1).split(1 << 28))
                info["full_size_checksum_equal"] = tot == ref
                info["pass"] = info["oracle_exact"] and info["full_size_checksum_equal"]
            else:
                okv = u.fp_close(got, exp)
                info["worst_rel_err_vs_fp64"] = u.worst_rel(got, exp)
                info["pass"] = bool(okv.all())
        else:
            # strided: fp64 reference over the whole matrix on the device (independent
            # implementation), plus the CPU oracle on the first 200k rows as its own problem
            x = buf.view(rows, cols)
            sample_sd = name.endswith("_sample")
            if name == "cfg3_mean":
                ref = x.mean(dim=0, dtype=torch.float64).cpu().numpy()
            else:
                m64 = x.mean(dim=0, dtype=torch.float64)
                ss = sum(((c.to(torch.float64) - m64) ** 2).sum(dim=0) for c in x.split(1 << 21))
                ref = torch.sqrt(ss / (rows - 1 if sample_sd else rows)).cpu().numpy()
            got = out_raw.view(torch.float32).cpu().numpy()
            info["worst_rel_err_vs_fp64_full"] = u.worst_rel(got, ref)
            ns = 200000
            sub = x[:ns].contiguous()
            d = api.make_desc(w["in_dt"], w["out_dt"], ns, cols, **{**kw, "final_scalar": 1.0 / ns})
            d.final_scalar = float(np.float32(1.0) / np.float32(ns - 1 if sample_sd else ns))
            if sample_sd:
                d.final_scalar2 = float(np.float32(d.final_scalar) * np.float32(ns))
            o = torch.zeros(cols, dtype=torch.float32, device=devc)
            auxs = None
            if w.get("needs_mean"):
                auxs = sub.mean(dim=0, dtype=torch.float64).to(torch.float32)
                d.final_aux = auxs.data_ptr()
            dev.reduce(d, sub, o)
            torch.cuda.synchronize()
            exp = u.oracle_reduce(d, sub.cpu().numpy().reshape(-1),
                                  aux=auxs.cpu().numpy().astype(np.float64) if auxs is not None else None)
            info["oracle_sample_rows"] = ns
            info["worst_rel_err_vs_fp64_sample"] = u.worst_rel(o.cpu().numpy(), exp)
            info["pass"] = bool(u.fp_close(got, ref).all() and u.fp_close(o.cpu().numpy(), exp).all())
        return info

    # ------------------------------------------------------------------
    # CPU baseline: the OpenMP host implementation on a bounded sample
    # ------------------------------------------------------------------
    def cpu_baseline(name, buf):
        from tests import _util as u
        w = WORK[name]
        rows, cols = w["rows"], w["cols"]
        es = api.DTYPE_SIZE[w["in_dt"]]
        cap_bytes = 512 << 20
        kw = dict(w["kw"])
        ns = min(rows, max(1, cap_bytes // (cols * es)))
        t = buf.view(rows, cols)[:ns].contiguous()
        host = (t.view(torch.int16).cpu().numpy().view(np.uint16) if w["in_dt"] == api.BF16
                else t.cpu().numpy()).reshape(-1)
        if "final_scalar" in kw and name.startswith("cfg3"):
            kw["final_scalar"] = float(np.float32(1.0) / np.float32(ns - 1 if name.endswith("_sample") else ns))
            if name.endswith("_sample"):
                kw["final_scalar2"] = float(np.float32(kw["final_scalar"]) * np.float32(ns))
        d = api.make_desc(w["in_dt"], w["out_dt"], ns, cols, **kw)
        no = ns if kw.get("apply", api.ALONG_ROWS) == api.ALONG_ROWS else cols
        out = np.zeros(no, dtype=u.out_numpy_dtype(w["out_dt"]))
        auxh = np.full(no, 3.0, dtype=np.float32) if w.get("needs_mean") else None
        threads = u.load_oracle().orc_max_threads()
        try:
            threads = min(threads, len(os.sched_getaffinity(0)))
        except AttributeError:
            pass
        threads = max(1, threads)
        u.oracle_typed(d, host, out, aux=auxh, threads=threads)  # warm-up, first touch
        best = float("inf")
        for _ in range(5):
            t0 = time.perf_counter()
            u.oracle_typed(d, host, out, aux=auxh, threads=threads)
            best = min(best, time.perf_counter() - t0)
        nbytes = ns * cols * es + no * api.DTYPE_SIZE[w["out_dt"]]
        return dict(value=nbytes / best / 1e9, unit="GB/s", cores=threads, kind="port",
                    sample=f"{ns} of {rows} rows x {cols} cols ({nbytes / 1e6:.0f} MB), "
                           f"best of 5 after one warm-up, OpenMP schedule(static)",
                    rows_per_s=ns / best, seconds=best)

    # ------------------------------------------------------------------
    if args.only_kernel:
        for nm in args.only_kernel.split(","):
            run_config(nm, args.steps, args.warmup, check=False, extras=False)
            torch.cuda.empty_cache()
        if args.calib_copy:
            a = torch.empty(512 << 20, dtype=torch.uint8, device=devc).random_(0, 255)
            b = torch.empty_like(a)
            for _ in range(5):
                b.copy_(a)
            torch.cuda.synchronize()
        return

    def launch_floor_us():
        # the fixed cost of one launch: a reduction whose data is a few KB, same call path
        x = torch.zeros(64 * 64, dtype=torch.float32, device=devc)
        o = torch.zeros(64, dtype=torch.float32, device=devc)
        d = api.make_desc(api.F32, api.F32, 64, 64)
        ref = C.byref(d)
        for _ in range(20):
            lib.rmi_reduce(ref, x.data_ptr(), o.data_ptr(), None, 0, sptr)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(200):
            lib.rmi_reduce(ref, x.data_ptr(), o.data_ptr(), None, 0, sptr)
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / 200 * 1e3

    def extra_row_normalize(rows=1000000, cols=128):
        # the step after config 2 in an embedding pipeline: x / ||x||_2 per row, same
        # matrix shape; algorithmic bytes = matrix read once + written once.  With 129
        # columns the rows are no multiple of a cache line and the flat kernel takes them.
        xs = [mk_normal(rows, cols, 2 + 7919 * i) for i in range(3)]
        os_ = [torch.empty_like(x) for x in xs]
        d = api.make_desc(api.F32, api.F32, rows, cols, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
        ref = C.byref(d)
        call = lib.rmi_row_normalize
        for i in range(5):
            rc = call(ref, xs[i % 3].data_ptr(), os_[i % 3].data_ptr(), 1e-8, sptr)
            assert rc == 0, api.status_string(rc)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        n = max(10, args.steps // 4)
        e0.record(stream)
        for i in range(n):
            call(ref, xs[i % 3].data_ptr(), os_[i % 3].data_ptr(), 1e-8, sptr)
        e1.record(stream)
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / n
        nb = 2 * rows * cols * 4
        norms = torch.linalg.vector_norm(os_[0].view(rows, cols).double(), dim=1)
        return dict(workload=f"row_normalize L2 fp32 {rows}x{cols} (read + write)", ms_per_step=ms,
                    alg_bytes=nb, GBps=nb / (ms * 1e-3) / 1e9,
                    pct_of_peak=100.0 * nb / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS,
                    check={"unit_rows": bool(torch.allclose(norms, torch.ones_like(norms), atol=1e-6))})

    def extra_meanvar():
        # config 3's mean followed by stddev reads the matrix twice; meanvar gives the mean
        # and the variance in one read of the same 10000000x64 matrix
        rows, cols = 10000000, 64
        xs = [mk_normal(rows, cols, 3 + 7919 * i) for i in range(3)]
        mean = torch.empty(cols, dtype=torch.float32, device="cuda")
        var = torch.empty(cols, dtype=torch.float32, device="cuda")
        nws = lib.rmi_meanvar_workspace_bytes(api.F32, api.ROW_MAJOR, rows, cols)
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device="cuda")

        def call(i):
            return lib.rmi_meanvar(api.F32, api.ROW_MAJOR, rows, cols, 1, xs[i % 3].data_ptr(),
                                   mean.data_ptr(), var.data_ptr(), ws.data_ptr(), nws, sptr)
        for i in range(5):
            rc = call(i)
            assert rc == 0, api.status_string(rc)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        n = max(10, args.steps // 4)
        e0.record(stream)
        for i in range(n):
            call(i)
        e1.record(stream)
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / n
        nb = rows * cols * 4
        x = xs[(n - 1) % 3].view(rows, cols)
        ok = bool(torch.allclose(mean.double(), x.double().mean(dim=0), rtol=1e-5, atol=1e-5) and
                  torch.allclose(var.double(), x.double().var(dim=0, unbiased=True), rtol=1e-5))
        return dict(workload="meanvar fp32 10000000x64 row-major (one read)", ms_per_step=ms,
                    alg_bytes=nb, GBps=nb / (ms * 1e-3) / 1e9,
                    pct_of_peak=100.0 * nb / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS,
                    check={"torch_fp64": ok})

    def extra_wide_columns():
        # column sums over rows of 16 KB that are not whole vectors: every workgroup streams
        # whole adjacent rows (partials per workgroup, folded by the second launch)
        rows, cols = 32768, 4097
        xs = [mk_normal(rows, cols, 11 + 7919 * i) for i in range(3)]
        out = torch.empty(cols, dtype=torch.float32, device="cuda")
        d = api.make_desc(api.F32, api.F32, rows, cols, apply=api.ALONG_COLUMNS)
        ref = C.byref(d)
        nws = lib.rmi_reduce_workspace_bytes(ref)
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device="cuda")

        def call(i):
            return lib.rmi_reduce(ref, xs[i % 3].data_ptr(), out.data_ptr(), ws.data_ptr(), nws, sptr)
        for i in range(5):
            rc = call(i)
            assert rc == 0, api.status_string(rc)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        n = max(10, args.steps // 4)
        e0.record(stream)
        for i in range(n):
            call(i)
        e1.record(stream)
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / n
        nb = rows * cols * 4 + cols * 4
        want = xs[(n - 1) % 3].view(rows, cols).sum(dim=0, dtype=torch.float64)
        ok = bool(torch.allclose(out.double(), want, rtol=1e-5, atol=1e-5))
        return dict(workload="column sum fp32 32768x4097 (whole rows per workgroup)", ms_per_step=ms,
                    alg_bytes=nb, GBps=nb / (ms * 1e-3) / 1e9,
                    pct_of_peak=100.0 * nb / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS,
                    check={"torch_fp64": ok})

    def extra_dense_rows():
        # row sums over rows of 17 lane-loads with tail elements (66 floats): a workgroup's load
        # slots dealt over whole adjacent rows, the rows combined through LDS
        rows, cols = 2000000, 66
        xs = [mk_normal(rows, cols, 13 + 7919 * i) for i in range(3)]
        out = torch.empty(rows, dtype=torch.float32, device="cuda")
        d = api.make_desc(api.F32, api.F32, rows, cols)
        ref = C.byref(d)

        def call(i):
            return lib.rmi_reduce(ref, xs[i % 3].data_ptr(), out.data_ptr(), None, 0, sptr)
        for i in range(5):
            rc = call(i)
            assert rc == 0, api.status_string(rc)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        n = max(10, args.steps // 4)
        e0.record(stream)
        for i in range(n):
            call(i)
        e1.record(stream)
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / n
        nb = rows * cols * 4 + rows * 4
        want = xs[(n - 1) % 3].view(rows, cols).sum(dim=1, dtype=torch.float64)
        ok = bool(torch.allclose(out.double(), want, rtol=1e-5, atol=1e-5))
        return dict(workload="row sum fp32 2000000x66 (17 lane-loads with a tail, dense slots)",
                    ms_per_step=ms, alg_bytes=nb, GBps=nb / (ms * 1e-3) / 1e9,
                    pct_of_peak=100.0 * nb / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS,
                    check={"torch_fp64": ok})

    def extra_rows(rows, cols, what, l2=True):
        # L2 norms (or plain sums) of short or awkward rows: `what` names the kernel the planner takes
        xs = [mk_normal(rows, cols, 17 + 7919 * i) for i in range(3)]
        out = torch.empty(rows, dtype=torch.float32, device="cuda")
        d = (api.make_desc(api.F32, api.F32, rows, cols, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
             if l2 else api.make_desc(api.F32, api.F32, rows, cols))
        ref = C.byref(d)
        nws = lib.rmi_reduce_workspace_bytes(ref)
        ws = torch.empty(nws, dtype=torch.uint8, device="cuda") if nws else None

        def call(i):
            return lib.rmi_reduce(ref, xs[i % 3].data_ptr(), out.data_ptr(),
                                  ws.data_ptr() if nws else None, nws, sptr)
        for i in range(5):
            rc = call(i)
            assert rc == 0, api.status_string(rc)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        n = max(10, args.steps // 4)
        e0.record(stream)
        for i in range(n):
            call(i)
        e1.record(stream)
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / n
        nb = rows * cols * 4 + rows * 4
        x64 = xs[(n - 1) % 3].view(rows, cols).double()
        want = x64.pow(2).sum(dim=1).sqrt() if l2 else x64.sum(dim=1)
        ok = bool(torch.allclose(out.double(), want, rtol=1e-5, atol=1e-5 if l2 else 1e-2))
        return dict(workload=f"{'L2 row norm' if l2 else 'row sum'} fp32 {rows}x{cols} ({what})",
                    ms_per_step=ms, alg_bytes=nb, GBps=nb / (ms * 1e-3) / 1e9,
                    pct_of_peak=100.0 * nb / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS,
                    check={"torch_fp64": ok})

    def extra_cov():
        # covariance of config 3's matrix around its column means: the one contraction on the
        # path (matrix cores).  Two bounds: HBM (the matrix once + D^2 outputs) and the fp32
        # matrix peak (2 N D^2 flop, half of it by symmetry, at 157.3 TFLOP/s); the tighter one
        # (the longer time) is the roof.  `centered` times the reference's semantics (the call
        # leaves x - mu in the data: read + write).
        rows, cols = 10000000, 64
        xs = [mk_normal(rows, cols, 3 + 7919 * i, 3.0, 2.0) for i in range(3)]
        mus = [x.view(rows, cols).mean(dim=0, dtype=torch.float64).to(torch.float32) for x in xs]
        out = torch.empty(cols * cols, dtype=torch.float32, device="cuda")
        nws = lib.rmi_cov_workspace_bytes(api.F32, api.ROW_MAJOR, rows, cols)
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device="cuda")

        def call(i, flags):
            return lib.rmi_cov(api.F32, api.ROW_MAJOR, rows, cols, 1, flags, xs[i % 3].data_ptr(),
                               mus[i % 3].data_ptr(), out.data_ptr(), ws.data_ptr(), nws, sptr)
        res = {}
        n = max(10, args.steps // 4)
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        # Timing first, the fp64 check after it: a second of fp64 matrix products right before
        # the timed loop leaves the GPU at its power limit, and the loop then measures the
        # limiter (the same kernel 380 us per call before, 590 us after), not the kernel.
        for name, flags in (("read_only", 0), ("centered", api.COV_CENTER_DATA)):
            for i in range(10):
                rc = call(i, flags)
                assert rc == 0, api.status_string(rc)
            torch.cuda.synchronize()
            e0.record(stream)
            for i in range(n):
                call(i, flags)
            e1.record(stream)
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / n
            nb = rows * cols * 4 * (2 if flags else 1) + cols * cols * 4
            res[name] = dict(ms_per_step=ms, alg_bytes=nb, GBps=nb / (ms * 1e-3) / 1e9)
        # the centred loop left x - mu in the buffers: check a call on the third matrix regenerated
        del xs[:]
        fresh = mk_normal(rows, cols, 3 + 7919 * 2, 3.0, 2.0)
        rc = lib.rmi_cov(api.F32, api.ROW_MAJOR, rows, cols, 1, 0, fresh.data_ptr(), mus[2].data_ptr(),
                         out.data_ptr(), ws.data_ptr(), nws, sptr)
        assert rc == 0, api.status_string(rc)
        torch.cuda.synchronize()
        x = fresh.view(rows, cols)
        ref = torch.zeros(cols, cols, dtype=torch.float64, device="cuda")
        for c in x.split(1 << 20):
            d = (c - mus[2][None, :]).to(torch.float64)
            ref += d.T @ d
        ref /= rows - 1
        sc = torch.sqrt(torch.outer(torch.diagonal(ref), torch.diagonal(ref)))
        ok = bool(((out.view(cols, cols).double() - ref).abs() <= 1e-5 * sc).all())
        hbm_ms = (rows * cols * 4 + cols * cols * 4) / (PEAK_HBM_GBPS * 1e9) * 1e3
        mfma_ms = rows * cols * cols / 157.3e12 * 1e3
        ms = res["read_only"]["ms_per_step"]
        return dict(workload="stats::cov fp32 10000000x64 row-major around its column means",
                    ms_per_step=ms, alg_bytes=res["read_only"]["alg_bytes"],
                    GBps=res["read_only"]["GBps"],
                    pct_of_peak=100.0 * res["read_only"]["GBps"] / PEAK_HBM_GBPS,
                    bounds_ms={"hbm": hbm_ms, "mfma_fp32_symmetric": mfma_ms},
                    bound="hbm" if hbm_ms >= mfma_ms else "mfma",
                    frac_of_bound=max(hbm_ms, mfma_ms) / ms,
                    TFLOPs_symmetric=rows * cols * cols / (ms * 1e-3) / 1e12,
                    centered=res["centered"],
                    check={"torch_fp64": ok})

    results = {}
    cpu = {}
    for name in names:
        steps = args.steps
        res, bufs, outs = run_config(name, steps, args.warmup, check=not args.no_check)
        results[name] = res
        if not args.no_cpu:
            cpu[name] = cpu_baseline(name, bufs[0])
        del bufs, outs
        torch.cuda.empty_cache()

    head = results[HEADLINE]
    extras = ({"row_normalize": extra_row_normalize(), "row_normalize_129": extra_row_normalize(1000000, 129),
               "meanvar": extra_meanvar(),
               "wide_columns": extra_wide_columns(), "dense_rows": extra_dense_rows(),
               "rows_of_3": extra_rows(40000000, 3, "rows shorter than a vector, through LDS"),
               "rows_of_1100": extra_rows(120000, 1100, "one trip of five loads per thread"),
               "few_long_rows": extra_rows(525, 511305, "rows split: no partly filled last round of teams", l2=False),
               "cov": extra_cov()}
              if args.configs == "all" else {})
    # One short line: the contract's keys, and inside `roofline` / `config` / `cpu_baseline`
    # what a reader needs to recompute every workload's fraction (ms per step and
    # algorithmic bytes).  The long per-workload records go to a file beside the run.
    by_config = {}
    for name, r in list(results.items()) + list(extras.items()):
        by_config[name] = {"ms": round(r["ms_per_step"], 6), "alg_bytes": r["alg_bytes"],
                           "frac": round(r["GBps"] / PEAK_HBM_GBPS, 4),
                           "traffic": PROFILE_TRAFFIC.get(name),
                           "check": bool(all(v is True or not isinstance(v, bool)
                                             for v in (r.get("check") or {}).values()))}
        if "frac_of_bound" in r:
            by_config[name]["frac_of_bound"] = round(r["frac_of_bound"], 4)
            by_config[name]["bound"] = r["bound"]
    line = {
        "metric": "achieved HBM GB/s, L2 row norm fp32 1000000x128 (algorithmic bytes / kernel time)",
        "value": head["GBps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": WORK[HEADLINE]["desc"], "plan": head["plan"],
                   "buffers_rotated": head["buffers"], "timing": "hip events on the launch stream",
                   "generator": "splitmix64 counter-based (raft_amd/bench/synth.py); buffer i of a "
                                "workload uses seed + 7919 * i",
                   "seeds": {n: WORK[n]["seed"] for n in results}},
        "roofline": {"bound": "hbm", "achieved": head["GBps"], "peak": PEAK_HBM_GBPS,
                     "unit": "GB/s", "frac": head["GBps"] / PEAK_HBM_GBPS,
                     "traffic": PROFILE_TRAFFIC.get(HEADLINE),
                     "traffic_source": PROFILE_SOURCE,
                     "by_config": by_config},
        "cpu_baseline": dict(cpu.get(HEADLINE) or {},
                             by_config={n: round(c["value"], 2) for n, c in cpu.items()}) or None,
        "rows_per_s": head["rows_per_s"],
        "launch_floor_us": launch_floor_us(),
        "device": torch.cuda.get_device_name(0),
    }
    details = {"configs": results, "extras": extras, "cpu_baselines": cpu}
    for d in (ROOT / "gpurun_out", ROOT):
        try:
            if d.is_dir():
                with open(d / "bench_details.json", "w") as f:
                    json.dump(details, f, indent=1)
                line["details_file"] = str((d / "bench_details.json").relative_to(ROOT))
                break
        except OSError:
            continue
    print(json.dumps(line))


def _load_profile_traffic():
    """HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this program,
    scaled by the same counters' reading for a copy of known size: written by
    raft_amd/bench/profile_summary.py into profiles/traffic.json together with the commit the
    library was at.  Not measured in this run; None where the file has no entry."""
    path = ROOT / "profiles" / "traffic.json"
    try:
        with open(path) as f:
            doc = json.load(f)
    except (OSError, ValueError):
        return {}, "profiles/traffic.json missing"
    traffic = {k: v.get("hbm_bytes") for k, v in doc.get("configs", {}).items()}
    return traffic, f"profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE; commit {doc.get('commit', 'unknown')})"


PROFILE_TRAFFIC, PROFILE_SOURCE = _load_profile_traffic()


if __name__ == "__main__":
    main()
