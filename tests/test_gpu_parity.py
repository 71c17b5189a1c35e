"""GPU results through the C ABI against the CPU oracle on the same seeded inputs:
the shape grids of the reference's reduction tests, every launch plan, every dtype
pairing, inplace, unaligned inputs and empty inputs."""
import itertools

import numpy as np
import pytest

from raft_amd import _capi as api
from tests import _util as u

pytestmark = pytest.mark.gpu

LAYOUT_AXIS = list(itertools.product([api.ROW_MAJOR, api.COL_MAJOR],
                                     [api.ALONG_ROWS, api.ALONG_COLUMNS]))


def _rand(rng, dt, n, lo=-1.0, hi=1.0):
    if dt == api.F32:
        return rng.uniform(lo, hi, n).astype(np.float32)
    if dt == api.F64:
        return rng.uniform(lo, hi, n)
    if dt == api.F16:
        return rng.uniform(lo, hi, n).astype(np.float16)
    if dt == api.BF16:
        return u.to_bf16(rng.uniform(lo, hi, n).astype(np.float32))
    if dt == api.I8:
        return rng.integers(-128, 128, n, dtype=np.int8)
    if dt == api.U8:
        return rng.integers(0, 256, n, dtype=np.uint8)
    if dt == api.I32:
        return rng.integers(-100000, 100000, n, dtype=np.int32)
    if dt == api.I64:
        return rng.integers(-2**40, 2**40, n, dtype=np.int64)
    raise ValueError(dt)


# cpp/tests/linalg/reduce.cu:292-317: rows {11,1234} x cols {7,33,128,500}, 4 layout/axis
# combinations, sq_op / add_op / sqrt_op, inplace=false then inplace=true on the same
# output (:191-241).
@pytest.mark.parametrize("in_dt,out_dt", [(api.F32, api.F32), (api.F64, api.F64),
                                          (api.F32, api.F64)])
@pytest.mark.parametrize("rows,cols", itertools.product([11, 1234], [7, 33, 128, 500]))
def test_reduce_grid(gpu, in_dt, out_dt, rows, cols):
    rng = np.random.default_rng(1234)
    data = _rand(rng, in_dt, rows * cols)
    for layout, apply in LAYOUT_AXIS:
        d = api.make_desc(in_dt, out_dt, rows, cols, layout=layout, apply=apply,
                          main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
        first = u.check_against_oracle(d, data, label=f"{rows}x{cols} l{layout} a{apply}")
        d.inplace = 1
        u.check_against_oracle(d, data, old_raw=first,
                               label=f"{rows}x{cols} l{layout} a{apply} inplace")


# cpp/tests/linalg/reduce.cu:321-341 ("thick"): {3,9} x {17771,33333,100000}, float -> float,
# double -> double and float -> double, inplace = false then true (the reference runs row-major
# along rows; the other three layout / axis combinations ride along for float).
@pytest.mark.parametrize("in_dt,out_dt", [(api.F32, api.F32), (api.F64, api.F64), (api.F32, api.F64)])
@pytest.mark.parametrize("rows,cols", itertools.product([3, 9], [17771, 33333, 100000]))
def test_reduce_thick(gpu, in_dt, out_dt, rows, cols):
    rng = np.random.default_rng(1234)
    data = _rand(rng, in_dt, rows * cols)
    for layout, apply in LAYOUT_AXIS if in_dt == out_dt == api.F32 else [(api.ROW_MAJOR, api.ALONG_ROWS)]:
        d = api.make_desc(in_dt, out_dt, rows, cols, layout=layout, apply=apply,
                          main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
        first = u.check_against_oracle(d, data, label=f"thick {rows}x{cols} l{layout} a{apply}")
        d.inplace = 1
        u.check_against_oracle(d, data, old_raw=first,
                               label=f"thick {rows}x{cols} l{layout} a{apply} inplace")


# Many long rows: the automatic plan gives each row a team of 64, 128 or 256 threads
# depending on the row's length and the accumulator; lengths straddle the team sizes and
# leave ragged last batches and tail elements.  (1100 rows would leave a last round of 76
# wide teams: rows of four 64 KB pieces and more are split instead.)
@pytest.mark.parametrize("in_dt,out_dt,kw", [
    (api.F32, api.F32, dict(main_op=api.MAIN_SQ)),
    (api.F64, api.F64, {}),
    (api.BF16, api.F32, dict(main_op=api.MAIN_ABS)),
    (api.I8, api.I64, {}),
    (api.F32, api.KVP_I32_F32, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, init_f=-np.inf)),
    (api.F64, api.I64, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMIN, final_op=api.FIN_KEY,
                            init_f=np.inf)),
])
@pytest.mark.parametrize("rows,cols", [(3000, 1029), (3000, 2051), (2500, 4099), (2100, 8197),
                                       (2100, 16390), (1100, 33001)])
def test_many_long_rows(gpu, in_dt, out_dt, kw, rows, cols):
    rng = np.random.default_rng(rows + cols)
    data = _rand(rng, in_dt, rows * cols)
    d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
    p = api.plan_query(d)
    if rows == 1100 and p.kind == api.PLAN_ROW_SPLIT:
        assert p.blocks_per_out >= 3 and cols * api.DTYPE_SIZE[in_dt] >= 4 * 65536
    else:
        assert p.kind in (api.PLAN_ROW_WAVE, api.PLAN_ROW_BLOCK) and p.passes == 1
    u.check_against_oracle(d, data, label=f"long rows {rows}x{cols} dt{in_dt}")


def _same_with_zeroed_workspace(d, data, first, misalign_elems=0):
    """The same reduction with RMI_FLAG_WORKSPACE_ZEROED and a zeroed workspace (split rows
    then fold in the same launch where the ticket lines suffice): bit-identical, twice."""
    import torch
    d2 = api.ReduceDesc.from_buffer_copy(d)
    d2.flags = api.FLAG_WORKSPACE_ZEROED
    ws = torch.zeros(max(api.plan_query(d2).workspace_bytes, api.WORKSPACE_TICKET_BYTES),
                     dtype=torch.uint8, device="cuda")
    for _ in range(2):
        again = u.gpu_reduce(d2, data, misalign_elems=misalign_elems, workspace=ws)
        assert np.array_equal(np.asarray(first).view(np.uint8), np.asarray(again).view(np.uint8))


# Row counts that would leave a partly filled last round of wide teams: rows of four 64 KB
# pieces and more are split (with and without the single-launch fold), shorter ones get
# teams of half the width; row counts that fill their rounds stay whole.
@pytest.mark.parametrize("in_dt,out_dt,kw", [
    (api.F32, api.F32, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)),
    (api.BF16, api.F32, {}),
    (api.F64, api.F64, {}),
    (api.I8, api.I64, dict(main_op=api.MAIN_ABS)),
    (api.F32, api.KVP_I32_F32, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMIN, init_f=np.inf)),
])
@pytest.mark.parametrize("rows,row_bytes,kind,threads", [
    (525, 262144 + 52, api.PLAN_ROW_SPLIT, 256), (1100, 300000, api.PLAN_ROW_SPLIT, 256),
    (1800, 262144, api.PLAN_ROW_SPLIT, 256),
    (525, 140008, api.PLAN_ROW_BLOCK, 512), (1000, 140000, api.PLAN_ROW_BLOCK, 512),
    (1300, 100000, api.PLAN_ROW_BLOCK, 256), (2047, 70000, api.PLAN_ROW_BLOCK, 256),
    (512, 140000, api.PLAN_ROW_BLOCK, 1024), (1024, 300000, api.PLAN_ROW_BLOCK, 512),
    (1000, 300000, api.PLAN_ROW_BLOCK, 1024),
])
def test_tail_round_rows(gpu, in_dt, out_dt, kw, rows, row_bytes, kind, threads):
    es = api.DTYPE_SIZE[in_dt]
    cols = row_bytes // es
    rng = np.random.default_rng(rows + row_bytes + in_dt)
    data = _rand(rng, in_dt, rows * cols)
    d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
    p = api.plan_query(d)
    assert (p.kind, p.block_threads) == (kind, threads), (p.kind, p.block_threads, p.blocks_per_out)
    if kind == api.PLAN_ROW_SPLIT:
        assert 3 <= p.blocks_per_out <= 32
    first = u.check_against_oracle(d, data, label=f"tail round {rows}x{cols} dt{in_dt}")
    _same_with_zeroed_workspace(d, data, first)


# Long rows of 1- and 2-byte elements that start off a 32-bit word (odd lengths, inputs
# shifted by one to three elements): the team kernel reads them from their next whole word
# on and gives the elements before it to the row's first thread, whole rows and split ones,
# sums (tails cleared), maxima (tails duplicated) and element-wise tails alike.
@pytest.mark.parametrize("in_dt,out_dt,kw", [
    (api.BF16, api.F32, {}),
    (api.F16, api.F16, dict(main_op=api.MAIN_ABS, reduce_op=api.RED_MAX)),
    (api.BF16, api.BF16, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)),
    (api.I8, api.I64, dict(main_op=api.MAIN_SQ)),
    (api.I8, api.I32, dict(reduce_op=api.RED_MIN, init_i=127)),
    (api.U8, api.I64, {}),
    (api.BF16, api.KVP_I32_F32, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, init_f=-np.inf)),
])
@pytest.mark.parametrize("rows,cols,shift", [(37, 10531, 0), (37, 10531, 1), (300, 4689, 0), (64, 2071, 3),
                                             (5, 262145, 0), (3, 300001, 1), (2, 1000003, 2),
                                             (700, 70001, 0), (9, 1025, 1)])
def test_long_rows_off_words(gpu, in_dt, out_dt, kw, rows, cols, shift):
    rng = np.random.default_rng(rows + cols + shift + in_dt)
    data = _rand(rng, in_dt, rows * cols)
    d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
    first = u.check_against_oracle(d, data, misalign_elems=shift,
                                   label=f"off words {rows}x{cols} dt{in_dt} +{shift}")
    _same_with_zeroed_workspace(d, data, first, misalign_elems=shift)


# Rows that do not fill 128-byte lines, or that start off a line: the wave-per-row plan
# stages rows of whole 16-byte vectors through LDS (a line-aligned contiguous read of the
# wave's rows).  Row lengths that are multiples of 8 and 4 bytes only (they end in tail
# elements and take the direct path) sit beside them, so both sides of the plan's choice are
# covered.  Row counts leave partial last waves; shifts move the input by 16..112 bytes.
@pytest.mark.parametrize("in_dt,out_dt,kw,es", [
    (api.F32, api.F32, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT), 4),
    (api.F64, api.F64, {}, 8),
    (api.BF16, api.F32, {}, 2),
    (api.I8, api.I64, dict(main_op=api.MAIN_ABS), 1),
    (api.F32, api.KVP_I32_F32, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMIN, init_f=np.inf), 4),
])
@pytest.mark.parametrize("row_bytes", [272, 400, 516, 520, 528, 796, 800, 1000, 1200, 2052, 2064,
                                       4000, 4080, 4088, 4092])
@pytest.mark.parametrize("rows,shift", [(1, 0), (7, 16), (1000, 0), (1000, 112), (5003, 48)])
def test_staged_rows(gpu, in_dt, out_dt, kw, es, row_bytes, rows, shift):
    if row_bytes % es:
        pytest.skip("not a whole number of elements")
    cols = row_bytes // es
    rng = np.random.default_rng(row_bytes + rows + shift)
    data = _rand(rng, in_dt, rows * cols)
    d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
    assert api.plan_query(d).kind == api.PLAN_ROW_WAVE
    u.check_against_oracle(d, data, misalign_elems=shift // es,
                           label=f"staged {rows}x{cols} dt{in_dt} +{shift}")


# cpp/tests/linalg/coalesced_reduction.cu:109-139: 10000 x {3..270}, 10 x 25000, ...
@pytest.mark.parametrize("rows,cols", [(10000, c) for c in
                                       (3, 5, 7, 9, 17, 31, 32, 33, 55, 63, 64, 65, 128, 270)]
                         + [(10, 25000), (100, 4100), (1025, 2048), (5, 1 << 17)])
@pytest.mark.parametrize("dt", [api.F32, api.F64])
def test_coalesced_sweep(gpu, rows, cols, dt):
    rng = np.random.default_rng(rows * 131 + cols)
    data = _rand(rng, dt, rows * cols)
    d = api.make_desc(dt, dt, rows, cols, main_op=api.MAIN_SQ)
    first = u.check_against_oracle(d, data, label=f"coalesced {rows}x{cols}")
    d.inplace = 1
    u.check_against_oracle(d, data, old_raw=first, label=f"coalesced {rows}x{cols} inplace")


# cpp/tests/linalg/strided_reduction.cu:94-102: 1024 x {32,64,128,256}; plus odd widths.
@pytest.mark.parametrize("rows,cols", [(1024, c) for c in (32, 64, 128, 256)]
                         + [(4097, 3), (100000, 2), (33333, 20), (777, 1000), (50, 20000)])
@pytest.mark.parametrize("dt", [api.F32, api.F64])
def test_strided_sweep(gpu, rows, cols, dt):
    rng = np.random.default_rng(rows * 7 + cols)
    data = _rand(rng, dt, rows * cols)
    d = api.make_desc(dt, dt, rows, cols, apply=api.ALONG_COLUMNS, main_op=api.MAIN_SQ)
    first = u.check_against_oracle(d, data, label=f"strided {rows}x{cols}")
    d.inplace = 1
    u.check_against_oracle(d, data, old_raw=first, label=f"strided {rows}x{cols} inplace")


# Every row plan forced on a shape it applies to must agree with the oracle.
@pytest.mark.parametrize("plan", [api.PLAN_ROW_WAVE, api.PLAN_ROW_BLOCK, api.PLAN_ROW_SPLIT])
@pytest.mark.parametrize("rows,cols", [(37, 4096), (5, 70000), (300, 1000), (2, 262144 + 4)])
@pytest.mark.parametrize("in_dt,out_dt,red", [(api.F32, api.F32, api.RED_ADD),
                                              (api.F32, api.F32, api.RED_MAX),
                                              (api.I8, api.I64, api.RED_ADD),
                                              (api.F64, api.F64, api.RED_ADD)])
def test_forced_row_plans(gpu, plan, rows, cols, in_dt, out_dt, red):
    rng = np.random.default_rng(plan * 1000 + rows)
    data = _rand(rng, in_dt, rows * cols)
    init = {} if red == api.RED_ADD else dict(init_f=-np.inf)
    d = api.make_desc(in_dt, out_dt, rows, cols, reduce_op=red, plan_hint=plan, **init)
    u.check_against_oracle(d, data, label=f"plan {api.PLAN_NAME[plan]} {rows}x{cols}")


# Input / output type pairings and functor triples.
TYPE_CASES = [
    (api.I8, api.I64), (api.I8, api.I32), (api.U8, api.I64), (api.I32, api.I64),
    (api.I64, api.I64), (api.F16, api.F32), (api.F16, api.F16), (api.BF16, api.F32),
    (api.BF16, api.BF16), (api.I8, api.F16), (api.I8, api.F32), (api.I32, api.F64),
    (api.F32, api.F16), (api.F64, api.F32),
]


@pytest.mark.parametrize("in_dt,out_dt", TYPE_CASES)
@pytest.mark.parametrize("main", [api.MAIN_IDENTITY, api.MAIN_SQ, api.MAIN_ABS, api.MAIN_NZ])
def test_type_pairs_sum(gpu, in_dt, out_dt, main):
    rng = np.random.default_rng(in_dt * 100 + out_dt * 10 + main)
    for rows, cols, apply in [(257, 96, api.ALONG_ROWS), (64, 4096, api.ALONG_ROWS),
                              (3000, 8, api.ALONG_ROWS), (2000, 48, api.ALONG_COLUMNS)]:
        data = _rand(rng, in_dt, rows * cols)
        if out_dt == api.F16 and in_dt in (api.I8, api.I32):
            data = (data % 5).astype(data.dtype)  # keep sums inside f16's range
        d = api.make_desc(in_dt, out_dt, rows, cols, apply=apply, main_op=main)
        u.check_against_oracle(d, data, label=f"{api.DTYPE_NAME[in_dt]}->"
                               f"{api.DTYPE_NAME[out_dt]} main{main} {rows}x{cols}")


@pytest.mark.parametrize("in_dt,out_dt", [(api.F32, api.F32), (api.F64, api.F64),
                                          (api.F16, api.F32), (api.BF16, api.F32),
                                          (api.I8, api.I64), (api.I32, api.I32),
                                          (api.I64, api.I64), (api.U8, api.I32)])
@pytest.mark.parametrize("red", [api.RED_MAX, api.RED_MIN])
@pytest.mark.parametrize("main", [api.MAIN_IDENTITY, api.MAIN_ABS, api.MAIN_SQ])
def test_min_max(gpu, in_dt, out_dt, red, main):
    rng = np.random.default_rng(in_dt + 17 * red + 5 * main)
    big = 2**62
    for rows, cols, apply in [(129, 200, api.ALONG_ROWS), (7, 9000, api.ALONG_ROWS),
                              (5000, 4, api.ALONG_ROWS), (1500, 40, api.ALONG_COLUMNS)]:
        data = _rand(rng, in_dt, rows * cols)
        init = dict(init_f=-np.inf, init_i=-big) if red == api.RED_MAX else \
            dict(init_f=np.inf, init_i=big)
        d = api.make_desc(in_dt, out_dt, rows, cols, apply=apply, main_op=main, reduce_op=red,
                          **init)
        if out_dt == api.I32:
            d.init.i = -2**31 if red == api.RED_MAX else 2**31 - 1
        # identity / abs select one of the inputs: exact.  sq is squared in f64 and
        # rounded once to the output type.
        exact = out_dt in (api.F32, api.F64) and main != api.MAIN_SQ
        u.check_against_oracle(d, data, tol=0.0 if exact else None,
                               label=f"minmax {api.DTYPE_NAME[in_dt]} red{red} main{main}")


# NaN through max_op / min_op and the Linf norm: the reference's device max / min are fmax / fmin
# (core/math.hpp:375-397,517-533), which ignore NaN; a row of NaN only returns `init`.  NaN is
# scattered, fills whole rows and whole columns, and sits in the tail elements after the last
# whole 16-byte vector (the overlapping last lane-load sees those twice).  Every plan kind: rows
# inside a vector, one load per lane, lanes of a wave (direct and staged through LDS), teams,
# split rows with the second pass, and the column kernel with its second pass.  Checked against
# the oracle (exactly: max / min select one of the inputs) and against numpy's nanmax / nanmin.
NAN_SHAPES = [
    # rows, cols, apply, plan hint, expected plan kind
    (5000, 2, api.ALONG_ROWS, api.PLAN_ROW_LANES, api.PLAN_ROW_LANES),
    (5000, 3, api.ALONG_ROWS, api.PLAN_AUTO, api.PLAN_ROW_WAVE),      # rows through LDS
    (3000, 21, api.ALONG_ROWS, api.PLAN_AUTO, api.PLAN_ROW_WAVE),     # one load per lane, any G, tail
    (3000, 30, api.ALONG_ROWS, api.PLAN_AUTO, api.PLAN_ROW_WAVE),     # one load per lane, G = 8, tail
    (1000, 259, api.ALONG_ROWS, api.PLAN_AUTO, api.PLAN_ROW_WAVE),    # lanes of a wave, tail
    (1000, 200, api.ALONG_ROWS, api.PLAN_AUTO, api.PLAN_ROW_WAVE),    # staged through LDS
    (300, 4099, api.ALONG_ROWS, api.PLAN_AUTO, api.PLAN_ROW_BLOCK),   # teams, tail
    (37, 8197, api.ALONG_ROWS, api.PLAN_ROW_BLOCK, api.PLAN_ROW_BLOCK),
    (3, 300003, api.ALONG_ROWS, api.PLAN_AUTO, api.PLAN_ROW_SPLIT),   # split rows + second pass
    (5, 70001, api.ALONG_ROWS, api.PLAN_ROW_SPLIT, api.PLAN_ROW_SPLIT),
    (20000, 67, api.ALONG_COLUMNS, api.PLAN_AUTO, api.PLAN_COL_TILE),   # dense lanes, tail, 2 passes
    (30000, 64, api.ALONG_COLUMNS, api.PLAN_AUTO, api.PLAN_COL_TILE),
    (40000, 3, api.ALONG_COLUMNS, api.PLAN_AUTO, api.PLAN_COL_TILE),    # rows read in groups
    (700, 1001, api.ALONG_COLUMNS, api.PLAN_AUTO, api.PLAN_COL_TILE),
]


@pytest.mark.parametrize("in_dt,out_dt", [(api.F32, api.F32), (api.F64, api.F64), (api.F16, api.F32),
                                          (api.BF16, api.F32)])
@pytest.mark.parametrize("rows,cols,apply,hint,kind", NAN_SHAPES)
def test_max_min_ignore_nan(gpu, in_dt, out_dt, rows, cols, apply, hint, kind):
    import warnings
    rng = np.random.default_rng(rows * 31 + cols)
    m = rng.standard_normal((rows, cols))
    m[rng.random((rows, cols)) < 0.1] = np.nan
    m[rows // 3, :] = np.nan                       # a whole row
    m[:, cols // 2] = np.nan                       # a whole column
    m[min(rows - 1, 2), cols - 1] = np.nan         # the last element of a row: a tail element
    m[:, -1][rng.random(rows) < 0.5] = np.nan
    if in_dt == api.F32:
        data = m.astype(np.float32)
    elif in_dt == api.F64:
        data = m
    elif in_dt == api.F16:
        data = m.astype(np.float16)
    else:
        data = u.to_bf16(m.astype(np.float32).reshape(-1)).reshape(rows, cols)
    vals = u.from_bf16(data).astype(np.float64) if in_dt == api.BF16 else data.astype(np.float64)
    assert np.isnan(vals).sum() == np.isnan(m).sum()
    ax = 1 if apply == api.ALONG_ROWS else 0
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)
        cases = [(api.MAIN_IDENTITY, api.RED_MAX, -np.inf, np.nanmax(vals, axis=ax)),
                 (api.MAIN_IDENTITY, api.RED_MIN, np.inf, np.nanmin(vals, axis=ax)),
                 (api.MAIN_ABS, api.RED_MAX, 0.0, np.nanmax(np.abs(vals), axis=ax))]  # Linf norm
    for main, red, init, want in cases:
        want = np.where(np.isnan(want), init, want)
        d = api.make_desc(in_dt, out_dt, rows, cols, apply=apply, main_op=main, reduce_op=red,
                          init_f=init, plan_hint=hint)
        # two f64 fill a 16-byte vector: such rows take one lane each of the wave plan
        want_kind = api.PLAN_ROW_WAVE if kind == api.PLAN_ROW_LANES and in_dt == api.F64 else kind
        assert api.plan_query(d).kind == want_kind
        for shift in (0, 1):
            raw = u.check_against_oracle(d, data.reshape(-1), tol=0.0, misalign_elems=shift,
                                         label=f"nan {rows}x{cols} main{main} red{red} +{shift}")
            assert np.array_equal(raw.astype(np.float64), want), (main, red, shift)


# The same through the inplace merge and a 16-bit output: red(out_old, acc) must ignore a NaN
# on either side the way fmax / fmin do.
def test_max_nan_inplace_and_init(gpu):
    rows, cols = 64, 100
    m = np.full((rows, cols), np.nan, dtype=np.float32)
    m[1::2, 5] = 3.0
    d = api.make_desc(api.F32, api.F32, rows, cols, reduce_op=api.RED_MAX, init_f=-np.inf,
                      inplace=True)
    old = np.where(np.arange(rows) % 4 < 2, np.float32(np.nan), np.float32(7.0)).astype(np.float32)
    raw = u.check_against_oracle(d, m.reshape(-1), old_raw=old, tol=0.0, label="nan inplace")
    want = np.array([np.fmax(np.fmax(-np.inf, 3.0 if r % 2 else np.nan), old[r]) for r in range(rows)])
    assert np.array_equal(raw.astype(np.float64), want)


# Rounding of f32 / f64 results to 16-bit outputs, bit for bit: one-element rows make the
# output the conversion of the input itself.  torch's bfloat16 and numpy's float16 conversions
# are the independent statements of round-to-nearest-even; a truncating conversion fails on
# half of the values, a round-half-up one on the ties.
@pytest.mark.parametrize("out_dt", [api.BF16, api.F16])
def test_output_rounding_is_nearest_even(gpu, out_dt):
    import torch
    rng = np.random.default_rng(99)
    n = 1 << 20
    if out_dt == api.BF16:
        bits = rng.integers(0, 2**32, n, dtype=np.uint64).astype(np.uint32)
        bits[: n // 4] = (bits[: n // 4] & 0xFFFF0000) | 0x8000        # exact ties
        x = bits.view(np.float32)
        x = x[np.isfinite(x)]
        want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    else:
        x = (rng.standard_normal(n) * np.exp(rng.uniform(-12, 11, n))).astype(np.float32)
        h = x[: n // 4].astype(np.float16).astype(np.float32)           # exact ties: midpoints
        x[: n // 4] = (h + np.nextafter(h.astype(np.float16), np.float16(np.inf)).astype(np.float32)) / 2
        x = x[np.isfinite(x) & (np.abs(x) < 60000)]
        want = x.astype(np.float16).view(np.uint16)
    d = api.make_desc(api.F32, out_dt, x.size, 1)
    got = u.gpu_reduce(d, x).view(np.uint16)
    assert np.array_equal(got, want), np.flatnonzero(got != want)[:8]


# L1 / L2 / Linf norms (linalg/detail/norm.cuh:23-61), row and column, with and without sqrt;
# cpp/tests/linalg/norm.cu:238-306 (incl. half -> float).
@pytest.mark.parametrize("in_dt,out_dt", [(api.F32, api.F32), (api.F64, api.F64),
                                          (api.F16, api.F32)])
@pytest.mark.parametrize("norm", ["l1", "l2", "linf"])
@pytest.mark.parametrize("fin", [api.FIN_IDENTITY, api.FIN_SQRT])
def test_norms(gpu, in_dt, out_dt, norm, fin):
    rng = np.random.default_rng(42)
    main, red = {"l1": (api.MAIN_ABS, api.RED_ADD), "l2": (api.MAIN_SQ, api.RED_ADD),
                 "linf": (api.MAIN_ABS, api.RED_MAX)}[norm]
    for rows, cols in [(4, 8), (1024, 32), (1000, 100), (129, 1024), (37, 6000)]:
        data = _rand(rng, in_dt, rows * cols, -10, 10)
        for apply in (api.ALONG_ROWS, api.ALONG_COLUMNS):
            d = api.make_desc(in_dt, out_dt, rows, cols, apply=apply, main_op=main,
                              reduce_op=red, final_op=fin)
            u.check_against_oracle(d, data, label=f"{norm} {rows}x{cols} a{apply}")


# Key-value arg reductions: cpp/tests/linalg/reduce.cu:343-411 shapes, plus planted ties
# (lowest index must win), NaN (never wins), all -inf rows and signed zeros.
@pytest.mark.parametrize("in_dt,out_dt", [(api.F32, api.KVP_I32_F32), (api.F64, api.KVP_I32_F64),
                                          (api.F32, api.KVP_I64_F32), (api.F64, api.KVP_I64_F64),
                                          (api.F16, api.KVP_I32_F32), (api.BF16, api.KVP_I32_F32)])
@pytest.mark.parametrize("red", [api.RED_ARGMAX, api.RED_ARGMIN])
def test_kvp_arg_reduce(gpu, in_dt, out_dt, red):
    rng = np.random.default_rng(1234 + red)
    is_max = red == api.RED_ARGMAX
    for rows, cols in itertools.product([11, 1234], [7, 33, 128, 500]):
        data = _rand(rng, in_dt, rows * cols)
        d = api.make_desc(in_dt, out_dt, rows, cols, main_op=api.MAIN_KVP, reduce_op=red,
                          init_i=0, init_f=-np.inf if is_max else np.inf)
        first = u.check_against_oracle(d, data, label=f"kvp {rows}x{cols}")
        d.inplace = 1
        u.check_against_oracle(d, data, old_raw=first, label=f"kvp {rows}x{cols} inplace")
        # the reference's own init, {0, 0} (reduce.cu:360-385): a row whose values all lose
        # against 0 returns it
        d0 = api.make_desc(in_dt, out_dt, rows, cols, main_op=api.MAIN_KVP, reduce_op=red,
                           init_i=0, init_f=0.0)
        u.check_against_oracle(d0, data, label=f"kvp {rows}x{cols} init {{0, 0}}")


@pytest.mark.parametrize("plan", [api.PLAN_AUTO, api.PLAN_ROW_WAVE, api.PLAN_ROW_BLOCK,
                                  api.PLAN_ROW_SPLIT])
@pytest.mark.parametrize("cols", [64, 1000, 32000, 131072])
def test_argmax_ties_and_specials(gpu, plan, cols):
    rng = np.random.default_rng(cols)
    rows = 48
    m = rng.standard_normal((rows, cols)).astype(np.float32)
    for r in range(rows):
        kind = r % 6
        if kind == 0:      # exact ties of the maximum at 2..4 positions
            pos = rng.choice(cols, size=min(cols, 2 + r % 3), replace=False)
            m[r, pos] = m[r].max() + 1.0
        elif kind == 1:    # NaN scattered, never wins
            m[r, rng.choice(cols, size=min(cols, 5), replace=False)] = np.nan
        elif kind == 2:    # whole row -inf: init key wins
            m[r, :] = -np.inf
        elif kind == 3:    # signed zeros tie
            m[r, :] = -1.0
            pos = np.sort(rng.choice(cols, size=2, replace=False))
            m[r, pos[0]] = -0.0
            m[r, pos[1]] = 0.0
        elif kind == 4:    # constant row: index 0
            m[r, :] = 0.5
        # kind 5: plain random
    d = api.make_desc(api.F32, api.KVP_I32_F32, rows, cols, main_op=api.MAIN_KVP,
                      reduce_op=api.RED_ARGMAX, init_i=0, init_f=-np.inf, plan_hint=plan)
    raw = u.check_against_oracle(d, m.reshape(-1), label=f"ties cols={cols} plan={plan}")
    # independent of the oracle: numpy's first-maximum rule on rows without NaN
    for r in range(rows):
        if r % 6 != 1:
            assert int(raw["key"][r]) == int(np.argmax(m[r]))
    dk = api.make_desc(api.F32, api.I32, rows, cols, main_op=api.MAIN_KVP,
                       reduce_op=api.RED_ARGMAX, final_op=api.FIN_KEY, init_i=0,
                       init_f=-np.inf, plan_hint=plan)
    keys = u.gpu_reduce(dk, m.reshape(-1))
    assert np.array_equal(keys, raw["key"])


# Short rows (lane groups, the any-G and dense layouts, the overlapping last vector) scan a
# lane's batch from its highest index down with a shortened rule: ties inside and across
# vectors and in the row's tail, rows of NaN only, rows of the neutral value only (the lowest
# index below the init's key wins, core/operators.hpp:187-203 applied element after element),
# and an init whose key is not 0.
@pytest.mark.parametrize("in_dt,out_dt", [(api.F32, api.KVP_I32_F32), (api.F64, api.KVP_I64_F64),
                                          (api.BF16, api.KVP_I32_F32)])
@pytest.mark.parametrize("red", [api.RED_ARGMAX, api.RED_ARGMIN])
def test_arg_short_rows_specials(gpu, in_dt, out_dt, red):
    is_max = red == api.RED_ARGMAX
    worst = -np.inf if is_max else np.inf
    best = 100.0 if is_max else -100.0
    for cols in (5, 9, 17, 33, 37, 48, 62, 66, 100, 129, 130, 200, 300, 515, 1000):
        rng = np.random.default_rng(cols * 2 + int(is_max))
        rows = 700
        m = np.round(rng.standard_normal((rows, cols)) * 4).astype(np.float64)   # many ties
        for r in range(rows):
            kind = r % 10
            if kind == 0:      # the best value twice in the row's last elements
                m[r, cols - 1] = m[r, max(0, cols - 3)] = best
            elif kind == 1:    # ... in adjacent vectors
                c = int(rng.integers(0, cols))
                m[r, c] = m[r, min(cols - 1, c + 4)] = best
            elif kind == 2:    # NaN only: the init stays
                m[r, :] = np.nan
            elif kind == 3:    # the neutral value only: index 0 beats the init's key
                m[r, :] = worst
            elif kind == 4:    # NaN, then the neutral value from some index on
                c = int(rng.integers(0, cols))
                m[r, :c] = np.nan
                m[r, c:] = worst
            elif kind == 5:    # NaN scattered over ordinary values
                m[r, rng.random(cols) < 0.3] = np.nan
            elif kind == 6:    # the best value in the first and in the last element
                m[r, 0] = m[r, cols - 1] = best
        flat = m.reshape(-1)
        data = {api.F32: lambda: flat.astype(np.float32), api.F64: lambda: flat,
                api.BF16: lambda: u.to_bf16(flat.astype(np.float32))}[in_dt]()
        for init_i, init_f in ((0, worst), (7, worst), (3, 0.0)):
            d = api.make_desc(in_dt, out_dt, rows, cols, main_op=api.MAIN_KVP, reduce_op=red,
                              init_i=init_i, init_f=init_f)
            raw = u.check_against_oracle(d, data, label=f"arg specials {rows}x{cols} init {init_i}")
            if init_f == worst:
                keys = raw["key"]
                assert all(int(keys[r]) == init_i for r in range(2, rows, 10))          # NaN only
                assert all(int(keys[r]) == 0 for r in range(3, rows, 10))               # neutral only


# Arg reduction along the strided dimension (the reference restricts KVP outputs to the
# contiguous dimension, linalg/strided_reduction.cuh:70-77; here it is supported).
def test_kvp_strided(gpu):
    rng = np.random.default_rng(5)
    rows, cols = 3000, 24
    m = rng.standard_normal((rows, cols)).astype(np.float32)
    m[17, 3] = m[2900, 3] = 9.0
    d = api.make_desc(api.F32, api.KVP_I32_F32, rows, cols, apply=api.ALONG_COLUMNS,
                      main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, init_i=0, init_f=-np.inf)
    raw = u.check_against_oracle(d, m.reshape(-1), label="kvp strided")
    assert int(raw["key"][3]) == 17


# Columns walk their rows downwards with the shortened rule: ties between far rows, in the
# rows after the last whole tile and in one tile, columns of NaN only and of the neutral value
# only, an init whose key is not 0; narrow matrices, whole-row layouts and wide rows.
@pytest.mark.parametrize("in_dt,out_dt", [(api.F32, api.KVP_I32_F32), (api.F64, api.KVP_I64_F64)])
@pytest.mark.parametrize("red", [api.RED_ARGMAX, api.RED_ARGMIN])
@pytest.mark.parametrize("rows,cols", [(20011, 5), (9001, 33), (6007, 130), (2503, 600),
                                       (1201, 2049), (4099, 4100)])
def test_arg_columns_specials(gpu, in_dt, out_dt, red, rows, cols):
    is_max = red == api.RED_ARGMAX
    worst = -np.inf if is_max else np.inf
    best = 100.0 if is_max else -100.0
    rng = np.random.default_rng(rows + cols + int(is_max))
    m = np.round(rng.standard_normal((rows, cols)) * 4).astype(np.float64)   # many ties
    for c in range(cols):
        kind = c % 8
        if kind == 0:      # the best value in two far rows
            r = np.sort(rng.choice(rows, size=2, replace=False))
            m[r, c] = best
        elif kind == 1:    # ... in the last rows of the matrix
            m[rows - 1, c] = m[rows - 2, c] = best
        elif kind == 2:    # NaN only
            m[:, c] = np.nan
        elif kind == 3:    # the neutral value only
            m[:, c] = worst
        elif kind == 4:    # NaN, then the neutral value from some row on
            r = int(rng.integers(0, rows))
            m[:r, c] = np.nan
            m[r:, c] = worst
        elif kind == 5:    # NaN scattered
            m[rng.random(rows) < 0.3, c] = np.nan
        elif kind == 6:    # the best value in adjacent rows
            r = int(rng.integers(0, rows - 1))
            m[r, c] = m[r + 1, c] = best
    data = m.reshape(-1).astype(np.float32) if in_dt == api.F32 else m.reshape(-1)
    for init_i, init_f in ((0, worst), (7, worst)):
        d = api.make_desc(in_dt, out_dt, rows, cols, apply=api.ALONG_COLUMNS, main_op=api.MAIN_KVP,
                          reduce_op=red, init_i=init_i, init_f=init_f)
        raw = u.check_against_oracle(d, data, label=f"arg columns {rows}x{cols} init {init_i}")
        keys = raw["key"]
        assert all(int(keys[c]) == init_i for c in range(2, cols, 8))   # NaN only
        assert all(int(keys[c]) == 0 for c in range(3, cols, 8))        # the neutral value only


# Inputs whose device address is not 16-byte aligned take the element-wise load path.
@pytest.mark.parametrize("in_dt,out_dt", [(api.F32, api.F32), (api.I8, api.I64),
                                          (api.BF16, api.F32), (api.F64, api.F64)])
@pytest.mark.parametrize("rows,cols,apply", [(100, 256, api.ALONG_ROWS),
                                             (9, 40000, api.ALONG_ROWS),
                                             (2000, 8, api.ALONG_ROWS),
                                             (4000, 64, api.ALONG_COLUMNS)])
def test_unaligned_input(gpu, in_dt, out_dt, rows, cols, apply):
    rng = np.random.default_rng(3)
    data = _rand(rng, in_dt, rows * cols)
    d = api.make_desc(in_dt, out_dt, rows, cols, apply=apply)
    u.check_against_oracle(d, data, misalign_elems=1, label="unaligned")


# fp32 / int32 rows of whole vectors whose input starts off a 16-byte boundary are laid side by
# side in the wave, one load per lane (up to 32 lanes per row), so that a load instruction reads
# one contiguous span; the same shapes on a boundary, and their neighbours (tails, longer rows,
# arg-reductions, which keep the default layout), sit beside them.
@pytest.mark.parametrize("in_dt,out_dt,kw", [
    (api.F32, api.F32, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)),
    (api.F32, api.F64, {}),
    (api.I32, api.I64, dict(main_op=api.MAIN_ABS)),
    (api.F32, api.F32, dict(reduce_op=api.RED_MAX, init_f=-np.inf)),
    (api.F32, api.KVP_I32_F32, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMIN, init_f=np.inf)),
])
@pytest.mark.parametrize("cols", [36, 48, 64, 96, 100, 104, 124, 128, 132, 66])
@pytest.mark.parametrize("rows,shift", [(1, 1), (7, 2), (63, 3), (1000, 1), (5003, 2), (5003, 0), (4096, 5)])
def test_rows_off_a_vector_boundary(gpu, in_dt, out_dt, kw, cols, rows, shift):
    rng = np.random.default_rng(rows * 13 + cols + shift)
    data = _rand(rng, in_dt, rows * cols)
    d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
    assert api.plan_query(d).kind == api.PLAN_ROW_WAVE
    u.check_against_oracle(d, data, misalign_elems=shift,
                           label=f"off boundary {rows}x{cols} dt{in_dt} +{shift}")


# Empty extents: no rows -> nothing written; no columns -> final_op(init) per output
# (and red(old, init) when inplace).
def test_empty_inputs(gpu):
    data = np.zeros(0, dtype=np.float32)
    d = api.make_desc(api.F32, api.F32, 0, 128)
    assert u.gpu_reduce(d, data).size == 0
    d = api.make_desc(api.F32, api.F32, 5, 0, init_f=2.0, final_op=api.FIN_SQ)
    assert u.gpu_reduce(d, data).tolist() == [4.0] * 5
    d = api.make_desc(api.F32, api.F32, 5, 0, init_f=0.0, inplace=True)
    old = np.arange(5, dtype=np.float32)
    assert u.gpu_reduce(d, data, old_raw=old).tolist() == old.tolist()
    d = api.make_desc(api.F32, api.F32, 0, 7, apply=api.ALONG_COLUMNS, init_f=1.5)
    assert u.gpu_reduce(d, data).tolist() == [1.5] * 7
    di = api.make_desc(api.I8, api.I64, 3, 0, init_i=7)
    assert u.gpu_reduce(di, np.zeros(0, dtype=np.int8)).tolist() == [7, 7, 7]


# Mean with the reference's rounding of 1/N (stats/detail/mean.cuh:22,39), incl. the
# int8 -> half case of cpp/tests/stats/mean.cu:177-185.
@pytest.mark.parametrize("in_dt,out_dt", [(api.F32, api.F32), (api.F64, api.F64),
                                          (api.F16, api.F32), (api.I8, api.F16)])
@pytest.mark.parametrize("rows,cols", [(1024, 32), (1024, 64), (8000, 128), (20000, 2)])
@pytest.mark.parametrize("row_major", [True, False])
def test_mean(gpu, in_dt, out_dt, rows, cols, row_major):
    rng = np.random.default_rng(rows + cols)
    if in_dt == api.I8:
        data = rng.integers(-20, 30, rows * cols, dtype=np.int8)
    else:
        data = _rand(rng, in_dt, rows * cols, -3, 5)
    ratio = {api.F32: np.float32, api.F64: np.float64, api.F16: np.float16}[out_dt](1.0) / rows
    d = api.make_desc(in_dt, out_dt, rows, cols, apply=api.ALONG_COLUMNS,
                      layout=api.ROW_MAJOR if row_major else api.COL_MAJOR,
                      final_op=api.FIN_MUL_CONST, final_scalar=float(ratio))
    u.check_against_oracle(d, data, label="mean")


# Results do not depend on run-to-run scheduling: no atomics anywhere.
def test_bitwise_repeatable(gpu):
    rng = np.random.default_rng(9)
    for rows, cols, apply in [(4, 300000, api.ALONG_ROWS), (200000, 64, api.ALONG_COLUMNS),
                              (50000, 128, api.ALONG_ROWS)]:
        data = rng.standard_normal(rows * cols).astype(np.float32)
        d = api.make_desc(api.F32, api.F32, rows, cols, apply=apply)
        a = u.gpu_reduce(d, data)
        for _ in range(3):
            assert np.array_equal(a, u.gpu_reduce(d, data))


# Rows split over several workgroups, reduced in ONE launch: with RMI_FLAG_WORKSPACE_ZEROED the
# workgroup that finishes a row last folds its partials (in index order, so the result equals
# the two-launch plan's bit for bit) and its ticket wraps the row's ticket word back to zero.
# One zeroed workspace serves every call of the test, split and column plans mixed, shapes
# growing and shrinking; the ticket words must read zero after every call.
@pytest.mark.parametrize("in_dt,out_dt,kw", [
    (api.F32, api.F32, {}),
    (api.F32, api.F32, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)),
    (api.BF16, api.F32, {}),
    (api.F64, api.F64, {}),
    (api.F16, api.F16, dict(main_op=api.MAIN_ABS, reduce_op=api.RED_MAX)),
    (api.I8, api.I64, dict(main_op=api.MAIN_SQ)),
    (api.I32, api.I32, dict(reduce_op=api.RED_MIN, init_i=2**31 - 1)),
    (api.F32, api.KVP_I32_F32, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, init_f=-np.inf)),
    (api.F64, api.KVP_I64_F64, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMIN, init_f=np.inf)),
    (api.F32, api.F32, dict(inplace=True)),
])
def test_split_rows_single_launch(gpu, in_dt, out_dt, kw):
    import ctypes as C
    import torch
    lib = api.load()
    sptr = torch.cuda.current_stream().cuda_stream
    ws = torch.zeros(4 << 20, dtype=torch.uint8, device="cuda")   # zeroed once, then only reused
    scratch = torch.empty(4 << 20, dtype=torch.uint8, device="cuda")
    rng = np.random.default_rng(in_dt * 7 + out_dt)
    odt = u.out_numpy_dtype(out_dt)
    # (the last three: two levels of counters with about a hundred rows, and more than sixteen
    # groups of sixteen chunks per row)
    shapes = [(8, 300_001, api.PLAN_AUTO), (1, 2_000_000, api.PLAN_AUTO), (3, 70_001, api.PLAN_ROW_SPLIT),
              (40, 80_000, api.PLAN_ROW_SPLIT), (2, 1_000_003, api.PLAN_AUTO), (512, 70_000, api.PLAN_ROW_SPLIT),
              (5, 100_003, api.PLAN_ROW_SPLIT), (100, 200_003, api.PLAN_ROW_SPLIT),
              (96, 150_000, api.PLAN_AUTO), (1, 6_000_001, api.PLAN_AUTO)]
    for rows, cols, hint in shapes:
        data = _rand(rng, in_dt, rows * cols)
        x = torch.from_numpy(data.view(np.uint8).reshape(-1)).cuda()
        old = u.encode_out(out_dt, rng.integers(-3, 4, rows).astype(np.float64)) if kw.get("inplace") else None
        outs = []
        for flags in (api.FLAG_WORKSPACE_ZEROED, 0):
            d = api.make_desc(in_dt, out_dt, rows, cols, plan_hint=hint, flags=flags, **kw)
            pl = api.plan_query(d)
            assert pl.kind == api.PLAN_ROW_SPLIT and pl.passes == (1 if flags else 2), (rows, cols)
            assert pl.workspace_bytes <= ws.numel()
            for rep in range(2 if flags else 1):
                o = torch.zeros(rows * odt.itemsize, dtype=torch.uint8, device="cuda")
                if old is not None:
                    o.copy_(torch.from_numpy(old.view(np.uint8).reshape(-1)))
                w = ws if flags else scratch.random_(0, 255)
                rc = lib.rmi_reduce(C.byref(d), x.data_ptr(), o.data_ptr(), w.data_ptr(), w.numel(), sptr)
                assert rc == api.OK, api.status_string(rc)
                torch.cuda.synchronize()
                outs.append(o.cpu().numpy().view(odt).copy())
            if flags:
                assert int(ws[: api.WORKSPACE_TICKET_BYTES].max().item()) == 0, "tickets must wrap to zero"
        assert all(np.array_equal(outs[0].view(np.uint8), o.view(np.uint8)) for o in outs[1:]), (rows, cols)
        # and the oracle, at the usual bar
        d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
        got = u.decode_out(out_dt, outs[0])
        exp = u.oracle_reduce(d, data, old=u.decode_out(out_dt, old) if old is not None else None)
        if u.is_arg(d):
            assert np.array_equal(got[0], exp[0]) and np.array_equal(got[1], exp[1])
        elif out_dt in (api.I32, api.I64):
            assert np.array_equal(got, exp)
        elif out_dt in (api.F16, api.BF16):
            assert u.ulp16_ok(out_dt, outs[0], exp).all()
        else:
            assert u.fp_close(got, exp).all(), u.worst_rel(got, exp)
        # a column reduction through the same workspace in between leaves the tickets alone
        dc = api.make_desc(api.F32, api.F32, 5000, 64, apply=api.ALONG_COLUMNS,
                           flags=api.FLAG_WORKSPACE_ZEROED)
        xc = torch.ones(5000 * 64, device="cuda")
        oc = torch.zeros(64, device="cuda")
        assert lib.rmi_reduce(C.byref(dc), xc.data_ptr(), oc.data_ptr(), ws.data_ptr(), ws.numel(), sptr) == api.OK
        torch.cuda.synchronize()
        assert bool((oc == 5000).all()) and int(ws[: api.WORKSPACE_TICKET_BYTES].max().item()) == 0


# Ticket words that were left non-zero (here: random bytes) are recovered by rmi_workspace_reset,
# a kernel on the caller's stream; rmi_noalloc_reset does the same for the static buffer.
def test_workspace_reset_recovers_ticket_words(gpu):
    import ctypes as C
    import torch
    lib = api.load()
    sptr = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(77)
    rows, cols = 6, 400_003
    data = rng.uniform(-1, 1, rows * cols).astype(np.float32)
    x = torch.from_numpy(data).cuda()
    d0 = api.make_desc(api.F32, api.F32, rows, cols)
    want = u.gpu_reduce(d0, data)
    df = api.make_desc(api.F32, api.F32, rows, cols, flags=api.FLAG_WORKSPACE_ZEROED)
    assert api.plan_query(df).passes == 1
    ws = torch.empty(1 << 20, dtype=torch.uint8, device="cuda").random_(1, 255)
    assert lib.rmi_workspace_reset(ws.data_ptr(), ws.numel(), sptr) == api.OK
    assert int(ws[: api.WORKSPACE_TICKET_BYTES].max().item()) == 0
    assert int(ws[api.WORKSPACE_TICKET_BYTES:].min().item()) >= 1   # nothing past the ticket words
    for _ in range(2):
        out = torch.zeros(rows, device="cuda")
        assert lib.rmi_reduce(C.byref(df), x.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel(), sptr) == api.OK
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), want)
    # a short workspace is cleared whole, nothing beyond it
    small = torch.empty(4096, dtype=torch.uint8, device="cuda").random_(1, 255)
    assert lib.rmi_workspace_reset(small.data_ptr(), 1024, sptr) == api.OK
    torch.cuda.synchronize()
    assert int(small[:1024].max().item()) == 0 and int(small[1024:].min().item()) >= 1
    assert lib.rmi_workspace_reset(None, 0, sptr) == api.OK
    assert lib.rmi_workspace_reset(None, 16, sptr) == api.ERR_NULL
    assert lib.rmi_workspace_reset(small.data_ptr() + 4, 16, sptr) == api.ERR_WORKSPACE
    # the static buffer of rmi_reduce_noalloc
    assert lib.rmi_noalloc_reset(sptr) == api.OK
    out = torch.zeros(rows, device="cuda")
    assert lib.rmi_reduce_noalloc(C.byref(d0), x.data_ptr(), out.data_ptr(), sptr) == api.OK
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), want)


# More rows than ticket words: the plan falls back to the folding launch.
def test_split_rows_beyond_the_ticket_words(gpu):
    d = api.make_desc(api.F32, api.F32, 513, 9000, plan_hint=api.PLAN_ROW_SPLIT,
                      flags=api.FLAG_WORKSPACE_ZEROED)
    assert api.plan_query(d).passes == 2
    rng = np.random.default_rng(1)
    u.check_against_oracle(d, _rand(rng, api.F32, 513 * 9000), label="split, two launches")


# Column reductions over rows that are not a power-of-two number of lane-loads: a workgroup
# takes as many whole rows as fit its 256 threads and combines them through LDS.  Rows shorter
# than a 16-byte vector are read in groups of 2..16 consecutive rows that make whole vectors
# (each real column then gets group x blocks partials, and the rows after the last whole
# group are added element by element); a start off a 16-byte boundary and arg-reductions
# read such rows element by element instead, with the same result.
@pytest.mark.parametrize("in_dt,out_dt,kw", [
    (api.F32, api.F32, {}),
    (api.F32, api.F32, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)),
    (api.F32, api.F32, dict(reduce_op=api.RED_MAX, init_f=-np.inf)),
    (api.F64, api.F64, {}),
    (api.BF16, api.F32, {}),
    (api.F16, api.F32, dict(main_op=api.MAIN_ABS)),
    (api.I8, api.I64, {}),
    (api.I32, api.I64, dict(reduce_op=api.RED_MIN, init_i=2**62)),
    (api.F32, api.KVP_I32_F32, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, init_f=-np.inf)),
])
@pytest.mark.parametrize("rows,cols", [(1024, 3), (70001, 3), (1027, 5), (300000, 7), (4099, 63),
                                       (70001, 129), (5000, 130), (2051, 1001), (66000, 33),
                                       (530, 4097), (255, 63), (40000, 1), (33333, 2),
                                       (9000, 100), (3000, 260), (2500, 517), (77, 37)])
@pytest.mark.parametrize("shift", [0, 1])
def test_grouped_columns(gpu, in_dt, out_dt, kw, rows, cols, shift):
    es = api.load().rmi_dtype_size(in_dt)
    rng = np.random.default_rng(rows * 7 + cols + shift)
    data = _rand(rng, in_dt, rows * cols)
    d = api.make_desc(in_dt, out_dt, rows, cols, apply=api.ALONG_COLUMNS, **kw)
    pl = api.plan_query(d)
    assert pl.kind == api.PLAN_COL_TILE
    if cols * es < 16 and kw.get("main_op") != api.MAIN_KVP and rows >= 4096:
        group = 16 // np.gcd(16, cols * es)
        assert pl.passes == 2 and pl.blocks_per_out % group == 0
    u.check_against_oracle(d, data, misalign_elems=shift,
                           label=f"grouped {rows}x{cols} dt{in_dt} +{shift}")


# Rows of 16 bytes or more that are 1 or 2 bytes off whole words (odd byte counts, odd counts of
# 16-bit elements) are read in groups of 16 or 8 as well up to 130 bytes:
# every row count around a whole group, sums, extrema and squares, in place.
@pytest.mark.parametrize("in_dt,out_dt,kw", [
    (api.BF16, api.F32, {}),
    (api.F16, api.F32, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)),
    (api.BF16, api.BF16, dict(reduce_op=api.RED_MAX, init_f=-np.inf)),
    (api.I8, api.I64, {}),
    (api.U8, api.I32, dict(main_op=api.MAIN_SQ)),
    (api.I8, api.F32, dict(main_op=api.MAIN_ABS)),
    (api.I8, api.I32, dict(reduce_op=api.RED_MIN, init_i=127)),
])
@pytest.mark.parametrize("cols", [9, 17, 33, 65, 127])
def test_grouped_columns_off_words(gpu, in_dt, out_dt, kw, cols):
    es = api.load().rmi_dtype_size(in_dt)
    rb = cols * es
    group = 16 // np.gcd(16, rb)
    for rows in [4096 + k for k in (0, 1, group - 1, group, group + 1)] + [50007]:
        rng = np.random.default_rng(rows * 3 + cols)
        data = _rand(rng, in_dt, rows * cols)
        d = api.make_desc(in_dt, out_dt, rows, cols, apply=api.ALONG_COLUMNS, **kw)
        pl = api.plan_query(d)
        assert pl.kind == api.PLAN_COL_TILE
        if 16 < rb <= 130 and rb % 4 != 0:
            assert pl.passes == 2 and pl.blocks_per_out % group == 0, (rows, cols, pl.blocks_per_out)
        first = u.check_against_oracle(d, data, label=f"grouped off words {rows}x{cols} dt{in_dt}")
        d.inplace = 1
        u.check_against_oracle(d, data, old_raw=first, label=f"grouped off words {rows}x{cols} dt{in_dt} inplace")
        d.inplace = 0
        u.check_against_oracle(d, data, misalign_elems=1, label=f"grouped off words {rows}x{cols} dt{in_dt} +1")


# Rows of 257 to 2304 lane-loads are read by a team in ONE trip of up to nine loads per thread
# (positions past the row re-read its last vector), the overlapping last vector among them: row
# lengths around every boundary of the rule, with and without tail elements, few rows (wider
# teams) and enough rows to fill the machine (the narrowest team), sums, extrema, arg-reductions.
@pytest.mark.parametrize("in_dt,out_dt,kw", [
    (api.F32, api.F32, {}),
    (api.F32, api.F32, dict(reduce_op=api.RED_MAX, init_f=-np.inf)),
    (api.F32, api.KVP_I32_F32, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMIN, init_f=np.inf)),
    (api.F64, api.F64, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)),
    (api.BF16, api.F32, {}),
    (api.I8, api.I64, dict(main_op=api.MAIN_ABS)),
])
def test_team_rows_one_trip(gpu, in_dt, out_dt, kw):
    es = api.load().rmi_dtype_size(in_dt)
    vec = 16 // es
    seed = 0
    for nload in (257, 258, 300, 511, 512, 513, 576, 577, 1000, 1024, 1025, 1152, 1153, 2048, 2049, 2304, 2305):
        for short in (0, 1, vec - 1):                 # whole vectors, one element short, one element over
            cols = nload * vec - short
            for rows in (5, 2100):
                seed += 1
                rng = np.random.default_rng(seed)
                data = _rand(rng, in_dt, rows * cols)
                if kw.get("main_op") == api.MAIN_KVP:   # ties for the arg-reduction
                    data = np.round(data * 8).astype(data.dtype)
                d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
                first = u.check_against_oracle(d, data, label=f"one trip {rows}x{cols} dt{in_dt}")
                if seed % 4 == 0:
                    d.inplace = 1
                    u.check_against_oracle(d, data, old_raw=first, label=f"one trip {rows}x{cols} dt{in_dt} inplace")
                    d.inplace = 0
                if seed % 5 == 0:
                    u.check_against_oracle(d, data, misalign_elems=1, label=f"one trip {rows}x{cols} dt{in_dt} +1")


# Rows through LDS: a workgroup reads a chunk of whole rows as aligned vectors and its threads
# reduce whole rows element by element.  Rows shorter than a vector, 16-bit and 8-byte rows
# that are no whole vectors, short fp32 rows; row counts around a chunk, matrices that end
# inside a vector, every reduction, in place, an input off a 16-byte boundary (other plans).
@pytest.mark.parametrize("in_dt,out_dt,kw,colset", [
    (api.F32, api.F32, {}, (3, 5, 6, 7, 9, 10)),
    (api.F32, api.F32, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT), (3, 9)),
    (api.F32, api.KVP_I32_F32, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, init_f=-np.inf), (3, 7)),
    (api.F32, api.F32, dict(reduce_op=api.RED_MIN, init_f=np.inf), (3, 10)),
    (api.F64, api.F64, {}, (3, 5, 9, 33, 63)),
    (api.F64, api.KVP_I64_F64, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMIN, init_f=np.inf), (3, 17)),
    (api.BF16, api.F32, {}, (3, 5, 7, 9, 17, 33, 100, 129, 255)),
    (api.F16, api.F16, dict(main_op=api.MAIN_ABS, reduce_op=api.RED_MAX, init_f=0.0), (3, 11, 65)),
    (api.I8, api.I64, {}, (3, 5, 7, 11, 15)),
    (api.U8, api.I32, dict(main_op=api.MAIN_SQ), (6, 13)),
    (api.I8, api.F32, dict(main_op=api.MAIN_NZ), (9,)),
    (api.I32, api.I64, {}, (3, 6)),
])
def test_small_rows_through_lds(gpu, in_dt, out_dt, kw, colset):
    es = api.load().rmi_dtype_size(in_dt)
    seed = 0
    for cols in colset:
        chunk = 16384 // (cols * es) // 16 * 16
        for rows in sorted({1, 2, 15, 16, 17, chunk - 1, chunk, chunk + 1, 2 * chunk + 3, 50001}):
            seed += 1
            rng = np.random.default_rng(seed * 11 + in_dt)
            data = _rand(rng, in_dt, rows * cols)
            if kw.get("main_op") == api.MAIN_KVP:       # ties
                data = np.round(data * 4).astype(data.dtype)
            d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
            pl = api.plan_query(d)
            assert pl.kind == api.PLAN_ROW_WAVE and pl.passes == 1
            assert pl.grid_blocks == -(-rows // chunk), (rows, cols, pl.grid_blocks)
            first = u.check_against_oracle(d, data, label=f"small rows {rows}x{cols} dt{in_dt}")
            if seed % 3 == 0:
                d.inplace = 1
                u.check_against_oracle(d, data, old_raw=first, label=f"small rows {rows}x{cols} dt{in_dt} inplace")
                d.inplace = 0
            if seed % 4 == 0:
                u.check_against_oracle(d, data, misalign_elems=1, label=f"small rows {rows}x{cols} dt{in_dt} +1")


# Byte rows that are no whole 32-bit words (17 to 96 bytes) are summed by the flat kernel:
# the matrix as one run of aligned 16-byte vectors, a vector's two row parts folded through
# LDS.  Row counts around the chunk sizes, matrices whose last vector is a partial one (it is
# read as the 16 bytes that end at the matrix's end), every output type, in place.
@pytest.mark.parametrize("in_dt", [api.I8, api.U8])
@pytest.mark.parametrize("out_dt,main", [(api.I64, api.MAIN_IDENTITY), (api.I32, api.MAIN_SQ),
                                         (api.F32, api.MAIN_ABS), (api.I64, api.MAIN_NZ)])
def test_flat_byte_rows(gpu, in_dt, out_dt, main):
    seed = 0
    for cols in (17, 18, 19, 21, 33, 47, 50, 65, 70, 85, 95):
        chunk = 16272 // cols
        for rows in sorted({1, 2, 15, 16, 17, chunk - 1, chunk, chunk + 1, 3 * chunk + 5, 40009}):
            seed += 1
            rng = np.random.default_rng(seed * 7 + in_dt)
            data = _rand(rng, in_dt, rows * cols)
            d = api.make_desc(in_dt, out_dt, rows, cols, main_op=main)
            pl = api.plan_query(d)
            assert pl.kind == api.PLAN_ROW_WAVE and pl.passes == 1
            first = u.check_against_oracle(d, data, label=f"flat bytes {rows}x{cols}")
            if seed % 3 == 0:
                d.inplace = 1
                u.check_against_oracle(d, data, old_raw=first, label=f"flat bytes {rows}x{cols} inplace")
            if seed % 5 == 0:  # off a 16-byte boundary: the lane-group plans take over
                d.inplace = 0
                u.check_against_oracle(d, data, misalign_elems=3, label=f"flat bytes {rows}x{cols} +3")



# Rows whose lane-load count suits neither a power-of-two lane group nor whole rows per wave
# (17, 18 or 33 lane-loads ending in tail elements; 16-bit rows of 9..16; compensated f64 sums
# of 5..18 or 34): a workgroup's load slots are dealt densely over whole adjacent rows and the
# rows are combined through LDS.  Row counts below one bundle, around one step, and beyond one
# round of the grid; starts off a 16-byte boundary; inplace.
@pytest.mark.parametrize("in_dt,out_dt,kw,cols_list", [
    (api.F32, api.F32, {}, (65, 66, 67, 69, 70, 71, 129, 130, 131)),
    (api.F32, api.F32, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT), (66, 129)),
    (api.F32, api.F32, dict(reduce_op=api.RED_MAX, init_f=-np.inf), (67, 131)),
    (api.F32, api.F16, dict(main_op=api.MAIN_ABS), (65,)),
    (api.BF16, api.F32, {}, (66, 76, 100, 127, 130, 132, 140, 260)),
    (api.F16, api.F32, dict(reduce_op=api.RED_MIN, init_f=np.inf), (73, 133, 259)),
    (api.F64, api.F64, {}, (9, 11, 17, 25, 33, 35, 65, 67)),
    (api.I8, api.I64, {}, (257, 270, 285, 520)),
    (api.U8, api.I32, {}, (260,)),
    (api.I32, api.I64, {}, (66, 129)),
    (api.F32, api.KVP_I32_F32, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, init_f=-np.inf),
     (65, 66, 70)),
    (api.F64, api.KVP_I64_F64, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMIN, init_f=np.inf),
     (33, 35)),
])
@pytest.mark.parametrize("rows,shift,inplace", [(1, 0, False), (7, 1, False), (29, 0, True), (121, 3, False),
                                                (1000, 0, False), (40003, 1, True), (150001, 0, False)])
def test_dense_rows(gpu, in_dt, out_dt, kw, cols_list, rows, shift, inplace):
    for cols in cols_list:
        rng = np.random.default_rng(rows * 13 + cols + shift)
        data = _rand(rng, in_dt, rows * cols)
        if kw.get("reduce_op") in (api.RED_MAX, api.RED_MIN):
            data[rng.integers(0, data.size, max(1, data.size // 50))] = np.nan
        if kw.get("main_op") == api.MAIN_KVP:  # ties: the lowest index has to win
            m = data.reshape(rows, cols)
            v = 9.0 if kw["reduce_op"] == api.RED_ARGMAX else -9.0
            m[:, cols - 1] = v
            m[:, cols // 2] = v
        d = api.make_desc(in_dt, out_dt, rows, cols, inplace=inplace, **kw)
        pl = api.plan_query(d)
        assert pl.kind == api.PLAN_ROW_WAVE and pl.passes == 1
        es = api.load().rmi_dtype_size(in_dt)
        if es in (2, 8) and cols * es <= 512 and (cols * es) % 16 != 0:
            # from a 16-byte boundary such rows go through LDS, a thread per row (the query's
            # answer); the dense slots serve them from any other start (shift != 0 below)
            assert pl.lanes_per_row == 1
        else:
            assert pl.lanes_per_row == -(-cols * es // 16), (cols, pl.lanes_per_row)
            assert pl.grid_blocks <= 4 * 256
        old = None
        if inplace and kw.get("main_op") != api.MAIN_KVP:
            old = u.encode_out(out_dt, rng.integers(1, 5, rows))
        elif inplace:
            continue
        u.check_against_oracle(d, data, misalign_elems=shift, old_raw=old,
                               label=f"dense rows {rows}x{cols} dt{in_dt} +{shift}")


# Column reductions over rows of more than 128 lane-loads that one workgroup can hold whole
# (floating sums, max and min): workgroups stream bundles of adjacent rows, one per CU, the
# rows of a bundle are combined through LDS and the partials [workgroup][column] are folded
# by a second launch.  Widths around the lane-load and slot boundaries, with and without
# tail elements; row counts from the fewest that take this plan, with rows left over after
# the last whole step; starts off a 16-byte boundary; both layouts; inplace.
def _whole_row_rows(lanes, slots_per_thread, bundles):
    """Fewest rows for which the planner streams whole rows: sixteen steps per workgroup."""
    n_cu = 256
    return n_cu * (256 * slots_per_thread // lanes) * bundles * 16


@pytest.mark.parametrize("in_dt,out_dt,kw,slots,bundles,cols_list", [
    (api.F32, api.F32, {}, 5, 2, (513, 516, 517, 700, 1024, 1025, 1300, 2049, 2560, 4097, 5119, 5120)),
    (api.F32, api.F32, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT), 5, 2, (1027, 4099)),
    (api.F32, api.F32, dict(reduce_op=api.RED_MAX, init_f=-np.inf), 5, 2, (519, 3001)),
    (api.F32, api.F16, dict(main_op=api.MAIN_ABS, final_op=api.FIN_MUL_CONST, final_scalar=1e-3), 5, 2, (2051,)),
    (api.F64, api.F64, {}, 5, 2, (257, 300, 513, 1025, 2049, 2560)),
    (api.F64, api.F64, dict(reduce_op=api.RED_MIN, init_f=np.inf), 5, 2, (301, 1281)),
    (api.BF16, api.F32, {}, 4, 3, (1025, 1030, 2056, 5500, 8191, 8192)),
    (api.F16, api.F32, dict(main_op=api.MAIN_ABS), 4, 3, (1100, 2741)),
    # byte sums: 32-bit slot accumulators, rows that fill three quarters of the 1024 slots
    (api.I8, api.I64, {}, 4, 3, (2100, 2730, 3000, 4100, 5000, 12300, 16000)),
    (api.I8, api.I32, dict(main_op=api.MAIN_SQ), 4, 3, (4100, 13000)),
    (api.U8, api.I64, dict(main_op=api.MAIN_NZ), 4, 3, (2500, 5001)),
    (api.I8, api.F32, dict(main_op=api.MAIN_ABS), 4, 3, (3001, 4100)),
    (api.U8, api.F16, dict(final_op=api.FIN_MUL_CONST, final_scalar=1e-4), 4, 3, (4099,)),
])
@pytest.mark.parametrize("extra,shift,col_major,inplace", [(0, 0, False, False), (37, 1, False, True),
                                                           (5, 0, True, False)])
def test_whole_row_columns(gpu, in_dt, out_dt, kw, slots, bundles, cols_list, extra, shift,
                           col_major, inplace):
    es = api.load().rmi_dtype_size(in_dt)
    for cols in cols_list:
        lanes = -(-cols * es // 16)
        rows = _whole_row_rows(lanes, slots, bundles) + extra
        rng = np.random.default_rng(cols * 3 + extra + shift)
        data = _rand(rng, in_dt, rows * cols)
        if kw.get("reduce_op") in (api.RED_MAX, api.RED_MIN):
            data[rng.integers(0, data.size, 5000)] = np.nan
            data.reshape(rows, cols)[:, 7] = np.nan  # a column of nothing but NaN keeps init
        if col_major:
            d = api.make_desc(in_dt, out_dt, cols, rows, layout=api.COL_MAJOR, apply=api.ALONG_ROWS,
                              inplace=inplace, **kw)
        else:
            d = api.make_desc(in_dt, out_dt, rows, cols, apply=api.ALONG_COLUMNS, inplace=inplace, **kw)
        pl = api.plan_query(d)
        assert pl.kind == api.PLAN_COL_TILE and pl.passes == 2
        assert pl.grid_blocks == 256 and pl.blocks_per_out == 256, (cols, pl.grid_blocks)
        _check_whole_rows(d, data, rng, cols, out_dt, shift, inplace)
        # one row fewer than the plan needs: the layout for short matrices, the same values
        if extra == 0 and cols == cols_list[0]:
            d2 = api.make_desc(in_dt, out_dt, rows - 1, cols, apply=api.ALONG_COLUMNS, **kw)
            assert api.plan_query(d2).grid_blocks != 256
            u.check_against_oracle(d2, data[:(rows - 1) * cols], label="one row fewer")


def _check_whole_rows(d, data, rng, cols, out_dt, shift, inplace):
    old = u.encode_out(out_dt, rng.uniform(1, 2, cols)) if inplace else None
    u.check_against_oracle(d, data, misalign_elems=shift, old_raw=old,
                           label=f"whole rows x{cols} dt{d.in_dtype} +{shift}")


# ... and rows that outgrow a workgroup's 1280 (16-bit elements: 1024) load slots, cut into the
# fewest equal pieces, 256 // pieces workgroups each: two to forty pieces, the last one shorter,
# with and without tail elements.  Rows that are whole multiples of 64 lane-loads keep the
# other layout.
@pytest.mark.parametrize("in_dt,out_dt,kw,slots,bundles,shapes", [
    (api.F32, api.F32, {}, 5, 2, ((5121, 2), (8191, 2), (11001, 3), (20003, 4), (50001, 10), (204700, 40))),
    (api.F32, api.F32, dict(reduce_op=api.RED_MIN, init_f=np.inf), 5, 2, ((6000, 2), (30000, 6))),
    (api.F64, api.F64, {}, 5, 2, ((2561, 2), (4097, 2), (12001, 5))),
    (api.BF16, api.F32, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT), 4, 3, ((10000, 2), (16400, 3))),
])
@pytest.mark.parametrize("extra,shift,inplace", [(0, 0, False), (3, 1, True)])
def test_whole_row_columns_in_pieces(gpu, in_dt, out_dt, kw, slots, bundles, shapes, extra, shift, inplace):
    es = api.load().rmi_dtype_size(in_dt)
    for cols, pieces in shapes:
        lanes = -(-cols * es // 16)
        piece = -(-lanes // pieces)
        b = 256 // pieces
        rows = b * (256 * slots // piece) * bundles * 16 + extra
        rng = np.random.default_rng(cols + extra)
        data = _rand(rng, in_dt, rows * cols)
        if kw.get("reduce_op") == api.RED_MIN:
            data[rng.integers(0, data.size, 5000)] = np.nan
        d = api.make_desc(in_dt, out_dt, rows, cols, apply=api.ALONG_COLUMNS, inplace=inplace, **kw)
        pl = api.plan_query(d)
        assert pl.kind == api.PLAN_COL_TILE and pl.passes == 2
        assert pl.blocks_per_out == b and pl.grid_blocks == b * pieces, (cols, pl.grid_blocks)
        _check_whole_rows(d, data, rng, cols, out_dt, shift, inplace)
    # whole multiples of 64 lane-loads in several pieces: not this plan
    d = api.make_desc(api.F32, api.F32, 4096, 32768, apply=api.ALONG_COLUMNS)
    assert api.plan_query(d).grid_blocks > 256


# Rows of 5 lane-loads, or of 6, 9..16, 18..21 and 28..32 with tail elements (up to 12 only for
# 16-byte accumulators): one lane per lane-load, 64 / G whole
# rows per wave step (G is not a power of two, the wave's last lanes idle).  Row counts around
# one wave's 4 * (64 / G) rows, and starts off a 16-byte boundary.
@pytest.mark.parametrize("in_dt,out_dt,kw,cols_list", [
    (api.F32, api.F32, {}, (17, 20, 21, 23, 33, 35, 38, 41, 45, 47, 50, 55, 59, 62, 70, 75, 79,
                            83, 110, 114, 118, 122, 125, 127)),
    (api.F32, api.F32, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT), (19, 34, 46)),
    (api.F64, api.F64, {}, (9, 10, 17, 19, 21, 23)),
    (api.BF16, api.F32, {}, (36, 70, 77, 85, 95, 100, 121)),
    (api.I8, api.I64, {}, (80, 131, 150, 170, 191)),
    (api.F32, api.KVP_I32_F32, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, init_f=-np.inf),
     (20, 33, 47)),
    (api.F32, api.F32, dict(reduce_op=api.RED_MIN, init_f=np.inf), (18, 43)),
])
@pytest.mark.parametrize("rows,shift", [(1, 0), (6, 1), (28, 0), (29, 3), (49, 0), (1000, 1), (5003, 0)])
def test_any_lane_count_rows(gpu, in_dt, out_dt, kw, cols_list, rows, shift):
    for cols in cols_list:
        rng = np.random.default_rng(rows * 11 + cols + shift)
        data = _rand(rng, in_dt, rows * cols)
        d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
        pl = api.plan_query(d)
        assert pl.kind == api.PLAN_ROW_WAVE
        # (from a 16-byte boundary the 16-bit and 8-byte shapes, and fp32 rows of up to 40 bytes,
        # go through LDS, a thread per row: the query answers 1 for them, and the lane groups
        # serve them from any other start, shift != 0)
        assert pl.lanes_per_row in (1, 5, 6) + tuple(range(9, 17)) + tuple(range(18, 22)) + tuple(range(28, 33)), \
            (cols, pl.lanes_per_row)
        u.check_against_oracle(d, data, misalign_elems=shift,
                               label=f"any-G {rows}x{cols} dt{in_dt} +{shift}")


# Column sums of 8-bit elements gather in 32-bit accumulators that are emptied into the
# 64-bit ones every 128 lane-loads: 17M rows give every thread of the 512 workgroups more
# than that.  Extreme values (all -128, squared) would overflow 32 bits within 2^17 terms.
@pytest.mark.parametrize("in_dt,kw", [(api.I8, dict(main_op=api.MAIN_SQ)), (api.U8, {}),
                                      (api.I8, dict(main_op=api.MAIN_ABS))])
def test_narrow_column_sums_many_rows(gpu, in_dt, kw):
    rows, cols = 17_000_001, 16
    npdt = np.int8 if in_dt == api.I8 else np.uint8
    data = np.full(rows * cols, -128 if in_dt == api.I8 else 255, dtype=npdt)
    rng = np.random.default_rng(5)
    idx = rng.integers(0, rows * cols, 1_000_000)
    data[idx] = rng.integers(-128 if in_dt == api.I8 else 0, 128 if in_dt == api.I8 else 256,
                             idx.size).astype(npdt)
    d = api.make_desc(in_dt, api.I64, rows, cols, apply=api.ALONG_COLUMNS, **kw)
    got = u.decode_out(api.I64, u.gpu_reduce(d, data))
    m = data.reshape(rows, cols).astype(np.int64)
    if kw.get("main_op") == api.MAIN_SQ:
        m = m * m
    elif kw.get("main_op") == api.MAIN_ABS:
        m = np.abs(m)
    assert np.array_equal(got, m.sum(axis=0))


# Rows that fit several times into one 16-byte vector (1, 2, 4 or 8 bytes long): lane-local
# sums, and each lane's results leave as one streamed 8- or 16-byte store when the epilogue is
# identity, sqrt or a multiplication by a constant and the output is f32, f64 or int64.
# Row counts that are not a multiple of the rows per vector end with lanes of their own.
@pytest.mark.parametrize("in_dt,out_dt,cols", [
    (api.F32, api.F32, 1), (api.F32, api.F32, 2), (api.F64, api.F64, 1), (api.BF16, api.F32, 1),
    (api.BF16, api.F32, 2), (api.F16, api.F32, 4), (api.F32, api.F64, 1), (api.F16, api.F64, 2),
    (api.I8, api.I64, 1), (api.I8, api.I64, 4), (api.U8, api.I64, 8), (api.I32, api.I64, 2),
    (api.I8, api.I32, 2),
])
@pytest.mark.parametrize("final", ["identity", "sqrt", "mul", "inplace"])
@pytest.mark.parametrize("rows", [1, 3, 1025, 70003])
def test_rows_inside_a_vector(gpu, in_dt, out_dt, cols, final, rows):
    integer = in_dt in (api.I8, api.U8, api.I32)
    if integer and final in ("sqrt", "mul"):
        pytest.skip("floating epilogues")
    kw = {}
    if final == "sqrt":
        kw = dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
    elif final == "mul":
        kw = dict(final_op=api.FIN_MUL_CONST, final_scalar=0.25)
    elif final == "inplace":
        kw = dict(inplace=True)
    rng = np.random.default_rng(rows + cols)
    data = _rand(rng, in_dt, rows * cols)
    old = None
    if final == "inplace":
        old = u.encode_out(out_dt, rng.integers(-5, 5, rows).astype(np.float64))
    # the plan asked for by name, and what the planner takes by itself (rows through LDS where
    # the output has 32 bits or more)
    d = api.make_desc(in_dt, out_dt, rows, cols, plan_hint=api.PLAN_ROW_LANES, **kw)
    assert api.plan_query(d).kind == api.PLAN_ROW_LANES
    u.check_against_oracle(d, data, old_raw=old, label=f"lanes {rows}x{cols} {final}")
    d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
    through_lds = api.load().rmi_dtype_size(out_dt) >= 4 and 16 // (cols * api.load().rmi_dtype_size(in_dt)) >= 4
    assert api.plan_query(d).kind == (api.PLAN_ROW_WAVE if through_lds else api.PLAN_ROW_LANES)
    u.check_against_oracle(d, data, old_raw=old, label=f"lanes or LDS {rows}x{cols} {final}")
