"""Randomised parity: seeded random shapes, layouts, axes, element types and functor
triples through the C ABI against the oracle.  The shape distribution is log-uniform in
both extents (up to a few million elements) and mixes in the values around which the plans
change (powers of two, one more, one less), so every plan and its edge cases are drawn."""
import os

import numpy as np
import pytest

from raft_amd import _capi as api
from tests import _util as u
from tests.test_gpu_parity import _rand

pytestmark = pytest.mark.gpu

SUM_TYPES = [(api.F32, api.F32), (api.F64, api.F64), (api.BF16, api.F32), (api.F16, api.F32),
             (api.I8, api.I64), (api.U8, api.I64), (api.I32, api.I64), (api.F32, api.F64),
             (api.I64, api.I64)]
MINMAX_TYPES = [(api.F32, api.F32), (api.F64, api.F64), (api.F16, api.F32), (api.I8, api.I64),
                (api.I32, api.I64)]
ARG_TYPES = [(api.F32, api.KVP_I32_F32), (api.F64, api.KVP_I32_F64), (api.F32, api.KVP_I64_F32),
             (api.BF16, api.KVP_I32_F32)]
EDGES = [1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257,
         511, 513, 1023, 1025, 4095, 4097]


def _extent(rng, cap):
    if rng.random() < 0.35:
        return int(min(cap, rng.choice(EDGES)))
    return int(min(cap, np.exp(rng.uniform(0, np.log(cap)))))


def _case(seed):
    rng = np.random.default_rng(seed)
    kind = rng.choice(["sum", "sum", "minmax", "arg"])
    total = 3_000_000
    a = _extent(rng, 300_000)
    b = _extent(rng, max(1, total // a))
    rows, cols = (a, b) if rng.random() < 0.5 else (b, a)
    layout = int(rng.choice([api.ROW_MAJOR, api.COL_MAJOR]))
    apply = int(rng.choice([api.ALONG_ROWS, api.ALONG_COLUMNS]))
    kw = dict(layout=layout, apply=apply)
    if kind == "sum":
        in_dt, out_dt = SUM_TYPES[rng.integers(len(SUM_TYPES))]
        kw["main_op"] = int(rng.choice([api.MAIN_IDENTITY, api.MAIN_SQ, api.MAIN_ABS, api.MAIN_NZ]))
        if out_dt in (api.F32, api.F64):
            fin = rng.choice(["id", "sqrt", "mul"])
            if fin == "sqrt" and kw["main_op"] in (api.MAIN_SQ, api.MAIN_ABS, api.MAIN_NZ):
                kw["final_op"] = api.FIN_SQRT
            elif fin == "mul":
                kw["final_op"], kw["final_scalar"] = api.FIN_MUL_CONST, 0.125
        if rng.random() < 0.25:
            kw["inplace"] = True
    elif kind == "minmax":
        in_dt, out_dt = MINMAX_TYPES[rng.integers(len(MINMAX_TYPES))]
        mx = rng.random() < 0.5
        kw["reduce_op"] = api.RED_MAX if mx else api.RED_MIN
        kw["main_op"] = int(rng.choice([api.MAIN_IDENTITY, api.MAIN_ABS]))
        kw["init_f"], kw["init_i"] = (-np.inf, -2**62) if mx else (np.inf, 2**62)
    else:
        in_dt, out_dt = ARG_TYPES[rng.integers(len(ARG_TYPES))]
        mx = rng.random() < 0.5
        kw.update(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX if mx else api.RED_ARGMIN,
                  init_f=-np.inf if mx else np.inf)
    es = api.DTYPE_SIZE[in_dt]
    shift = int(rng.choice([0, 0, 1, 2, 3, 16 // es if es < 16 else 1]))
    return kind, in_dt, out_dt, rows, cols, kw, shift, rng


# RMI_RANDOM_CASES widens the draw for a longer run
@pytest.mark.parametrize("seed", range(int(os.environ.get("RMI_RANDOM_CASES", "400"))))
def test_random_case(gpu, seed):
    kind, in_dt, out_dt, rows, cols, kw, shift, rng = _case(seed)
    data = _rand(rng, in_dt, rows * cols)
    if kind == "arg" and rows * cols > 8:
        # plant ties: copies of the extreme value at random places
        flat = data.reshape(-1)
        flat[rng.integers(0, flat.size, 6)] = flat.max() if kw["reduce_op"] == api.RED_ARGMAX \
            else flat.min()
    d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
    old = None
    if kw.get("inplace"):
        n = u.n_outputs(d)
        old = u.encode_out(out_dt, rng.integers(-3, 4, n).astype(np.float64))
    label = (f"seed {seed}: {kind} {api.DTYPE_NAME[in_dt]}->{api.DTYPE_NAME[out_dt]} {rows}x{cols} "
             f"layout {kw['layout']} apply {kw['apply']} +{shift} {kw}")
    raw = u.check_against_oracle(d, data, old_raw=old, misalign_elems=shift, label=label)
    if seed % 2 == 0:
        # every other case once more with RMI_FLAG_WORKSPACE_ZEROED through ONE workspace that
        # all such cases share (zeroed once, then only used by the library): the same bits
        _same_bits_with_shared_workspace(in_dt, out_dt, rows, cols, kw, data, old, shift, raw, label)


_shared = {}


def _shared_workspace():
    import torch
    if "ws" not in _shared:
        _shared["ws"] = torch.zeros(64 << 20, dtype=torch.uint8, device="cuda")
    return _shared["ws"]


def _same_bits_with_shared_workspace(in_dt, out_dt, rows, cols, kw, data, old, shift, raw, label):
    ws = _shared_workspace()
    df = api.make_desc(in_dt, out_dt, rows, cols, flags=api.FLAG_WORKSPACE_ZEROED, **kw)
    assert api.plan_query(df).workspace_bytes <= ws.numel(), label
    got = u.gpu_reduce(df, data, old_raw=old, misalign_elems=shift, workspace=ws)
    if got.dtype.names:   # key-value records: field by field (a record may hold padding bytes)
        same = all(np.array_equal(np.ascontiguousarray(got[f]).view(np.uint8),
                                  np.ascontiguousarray(raw[f]).view(np.uint8)) for f in got.dtype.names)
    else:
        same = np.array_equal(got.view(np.uint8), raw.view(np.uint8))
    assert same, f"{label}: the flagged plan differs from the plain one"
    assert int(ws[: api.WORKSPACE_TICKET_BYTES].max().item()) == 0, f"{label}: ticket words left non-zero"


# Rows long enough to be split over several workgroups are rare in the draw above: few rows of
# 70 thousand to 3 million elements, every accumulator family, counters in one level (up to
# 16 chunks per row) and in two, through the shared workspace with the flag and through a
# scratch one without it: the same bits, and the oracle's values.
@pytest.mark.parametrize("seed", range(int(os.environ.get("RMI_RANDOM_CASES", "400")) // 8))
def test_random_split_rows(gpu, seed):
    rng = np.random.default_rng(40_000 + seed)
    kind = rng.choice(["sum", "sum", "minmax", "arg"])
    rows = int(rng.choice([1, 1, 2, 3, 5, 8, 17, 40, 100]))
    cols = int(np.exp(rng.uniform(np.log(70_000), np.log(max(80_000, 4_000_000 // rows)))))
    cols += int(rng.integers(0, 9))
    kw = {}
    if kind == "sum":
        in_dt, out_dt = SUM_TYPES[rng.integers(len(SUM_TYPES))]
        kw["main_op"] = int(rng.choice([api.MAIN_IDENTITY, api.MAIN_SQ, api.MAIN_ABS]))
        kw["inplace"] = bool(rng.random() < 0.25)
    elif kind == "minmax":
        in_dt, out_dt = MINMAX_TYPES[rng.integers(len(MINMAX_TYPES))]
        mx = rng.random() < 0.5
        kw.update(reduce_op=api.RED_MAX if mx else api.RED_MIN,
                  init_f=-np.inf if mx else np.inf, init_i=-2**62 if mx else 2**62)
    else:
        in_dt, out_dt = ARG_TYPES[rng.integers(len(ARG_TYPES))]
        mx = rng.random() < 0.5
        kw.update(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX if mx else api.RED_ARGMIN,
                  init_f=-np.inf if mx else np.inf)
    hint = api.PLAN_ROW_SPLIT if rng.random() < 0.5 else api.PLAN_AUTO
    data = _rand(rng, in_dt, rows * cols)
    d = api.make_desc(in_dt, out_dt, rows, cols, plan_hint=hint, **kw)
    old = u.encode_out(out_dt, rng.integers(-3, 4, rows).astype(np.float64)) if kw.get("inplace") else None
    shift = int(rng.choice([0, 0, 1, 3]))
    label = f"seed {seed}: split rows {kind} {api.DTYPE_NAME[in_dt]}->{api.DTYPE_NAME[out_dt]} {rows}x{cols} +{shift} {kw}"
    raw = u.check_against_oracle(d, data, old_raw=old, misalign_elems=shift, label=label)
    _same_bits_with_shared_workspace(in_dt, out_dt, rows, cols, dict(kw, plan_hint=hint), data, old,
                                     shift, raw, label)


# The same for row normalisation and the one-pass mean / variance.
@pytest.mark.parametrize("seed", range(int(os.environ.get("RMI_RANDOM_CASES", "400")) // 4))
def test_random_normalize(gpu, seed):
    from tests import test_gpu_normalize as tn
    rng = np.random.default_rng(10_000 + seed)
    cols = _extent(rng, 100_000)
    rows = _extent(rng, max(1, 2_000_000 // cols))
    dt = int(rng.choice([api.F32, api.F32, api.F64, api.BF16, api.F16]))
    norm = str(rng.choice(list(tn.NORMS)))
    main, red, fin = tn.NORMS[norm]
    f = rng.uniform(-4, 4, rows * cols)
    if dt == api.BF16:
        data = u.to_bf16(f.astype(np.float32))
    else:
        data = f.astype({api.F32: np.float32, api.F64: np.float64, api.F16: np.float16}[dt])
    d = api.make_desc(dt, dt, rows, cols, main_op=main, reduce_op=red, final_op=fin)
    prev = np.zeros(rows * cols, dtype=data.dtype)
    raw = tn._gpu(d, data, prev, 1e-8)
    got = tn._as_f64(dt, raw)
    exp = tn._oracle(d, data, tn._as_f64(dt, prev), 1e-8)
    if dt in (api.F16, api.BF16):
        ok = u.ulp16_ok(dt, raw, exp)
    else:
        ok = u.approx_ok(got, exp, {api.F32: 1e-5, api.F64: 1e-8}[dt])
    assert ok.all(), (seed, dt, rows, cols, norm, u.worst_rel(got, exp))


@pytest.mark.parametrize("seed", range(int(os.environ.get("RMI_RANDOM_CASES", "400")) // 4))
def test_random_meanvar(gpu, seed):
    from tests import test_gpu_meanvar as tm
    rng = np.random.default_rng(20_000 + seed)
    a = _extent(rng, 200_000)
    b = _extent(rng, max(1, 2_000_000 // a))
    rows, cols = (a, b) if rng.random() < 0.5 else (b, a)
    dt = int(rng.choice([api.F32, api.F64]))
    layout = int(rng.choice([api.ROW_MAJOR, api.COL_MAJOR]))
    stored = tm._make(rng, dt, layout, rows, cols, float(rng.uniform(-50, 50)), float(rng.uniform(0.1, 5)))
    tm._check(dt, layout, rows, cols, bool(rng.random() < 0.5), stored)


# Column reductions of wide rows take their own layout only from a few hundred megabytes on
# (every workgroup has to get sixteen steps), which the draw above never reaches: random widths
# from 513 columns up to some hundred thousand, in one piece or several, with just enough rows
# for that layout plus a random remainder.
@pytest.mark.parametrize("seed", range(int(os.environ.get("RMI_RANDOM_CASES", "400")) // 10))
def test_random_wide_columns(gpu, seed):
    rng = np.random.default_rng(30_000 + seed)
    in_dt, out_dt = [(api.F32, api.F32), (api.F64, api.F64), (api.BF16, api.F32), (api.F16, api.F32),
                     (api.F32, api.F64)][rng.integers(5)]
    es = api.DTYPE_SIZE[in_dt]
    slots, bundles = (1024, 3) if es == 2 else (1280, 2)
    lanes = int(np.exp(rng.uniform(np.log(129), np.log(8 * slots))))
    cols = lanes * (16 // es) - int(rng.integers(0, 16 // es))
    lanes = -(-cols * es // 16)
    pieces = -(-lanes // slots)
    if pieces > 1 and lanes % 64 == 0 and cols * es % 16 == 0:
        cols -= 1                                   # rows of whole multiples of 64 lane-loads: other layout
        lanes = -(-cols * es // 16)
        pieces = -(-lanes // slots)
    piece = -(-lanes // pieces)
    b = 256 // pieces
    rows = b * (slots // piece) * bundles * 16 + int(rng.integers(0, 40))
    kw = {}
    op = rng.choice(["sum", "sq", "abs", "max", "min"])
    if op == "sq":
        kw.update(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
    elif op == "abs":
        kw.update(main_op=api.MAIN_ABS)
    elif op in ("max", "min"):
        kw.update(reduce_op=api.RED_MAX if op == "max" else api.RED_MIN,
                  init_f=-np.inf if op == "max" else np.inf)
    inplace = bool(rng.random() < 0.3)
    col_major = bool(rng.random() < 0.3)
    data = _rand(rng, in_dt, rows * cols)
    if col_major:
        d = api.make_desc(in_dt, out_dt, cols, rows, layout=api.COL_MAJOR, apply=api.ALONG_ROWS,
                          inplace=inplace, **kw)
    else:
        d = api.make_desc(in_dt, out_dt, rows, cols, apply=api.ALONG_COLUMNS, inplace=inplace, **kw)
    pl = api.plan_query(d)
    assert pl.kind == api.PLAN_COL_TILE and pl.passes == 2
    assert pl.blocks_per_out == b and pl.grid_blocks == b * pieces, (seed, rows, cols, pl.grid_blocks)
    old = u.encode_out(out_dt, rng.integers(-3, 4, cols).astype(np.float64)) if inplace else None
    shift = int(rng.choice([0, 0, 1, 3]))
    u.check_against_oracle(d, data, old_raw=old, misalign_elems=shift,
                           label=f"seed {seed}: wide columns {rows}x{cols} dt{in_dt}->{out_dt} {op} +{shift}")
