"""Pins the CPU oracle (oracle/oracle.cpp): every known-answer fixture the reference's
tests hold for the reduction path, plus closed forms and numpy routines on random
inputs chosen so that a dropped term, a wrong stride or a swapped axis fails."""
import itertools

import numpy as np
import pytest

from raft_amd import _capi as api
from tests import _util as u


GOLD = u.golden()


# cpp/tests/linalg/reduce.cu:108-177
@pytest.mark.parametrize("case", list(GOLD["reduce_simple_max"]["expected"]))
def test_simple_max_fixture(oracle, case):
    g = GOLD["reduce_simple_max"]
    layout, apply = u.LAYOUT_AXIS[case]
    expected = g["expected"][case]
    data = np.array(g["data"], dtype=np.float32)
    d = api.make_desc(api.F32, api.F32, g["rows"], g["cols"], layout=layout, apply=apply,
                      reduce_op=api.RED_MAX)
    assert u.oracle_reduce(d, data).tolist() == expected
    out = np.zeros(len(expected), dtype=np.float32)
    assert u.oracle_typed(d, data, out).tolist() == expected


# cpp/tests/matrix/argmax.cu:71-75, argmin.cu:71-75
def test_argmax_argmin_fixture(oracle):
    g = GOLD["matrix_arg"]
    data = np.array(g["data"], np.float32)
    d = api.make_desc(api.F32, api.I32, g["rows"], g["cols"], main_op=api.MAIN_KVP,
                      reduce_op=api.RED_ARGMAX, final_op=api.FIN_KEY, init_f=-np.inf)
    assert u.oracle_reduce(d, data)[0].tolist() == g["argmax"]
    out = np.zeros(g["rows"], dtype=np.int32)
    assert u.oracle_typed(d, data, out).tolist() == g["argmax"]
    d = api.make_desc(api.F32, api.I32, g["rows"], g["cols"], main_op=api.MAIN_KVP,
                      reduce_op=api.RED_ARGMIN, final_op=api.FIN_KEY, init_f=np.inf)
    assert u.oracle_reduce(d, data)[0].tolist() == g["argmin"]
    assert u.oracle_typed(d, data, out).tolist() == g["argmin"]


# cpp/tests/util/reduction.cu:167-171,179-181
def test_vector64_fixture(oracle):
    g = GOLD["wave_vector64"]
    x = np.array(g["data"], dtype=np.int32)
    for red, init, want in [(api.RED_MIN, 2**62, g["min"]), (api.RED_MAX, -2**62, g["max"]),
                            (api.RED_ADD, 0, g["sum"])]:
        d = api.make_desc(api.I32, api.I64, 1, 64, reduce_op=red, init_i=init)
        assert u.oracle_reduce(d, x).tolist() == [want]
    xf = x.astype(np.float32)
    d = api.make_desc(api.F32, api.KVP_I32_F32, 1, 64, main_op=api.MAIN_KVP,
                      reduce_op=api.RED_ARGMAX, init_f=-np.inf)
    k, v = u.oracle_reduce(d, xf)
    assert [k[0], v[0]] == g["argmax"]
    d = api.make_desc(api.F32, api.KVP_I32_F32, 1, 64, main_op=api.MAIN_KVP,
                      reduce_op=api.RED_ARGMIN, init_f=np.inf)
    k, v = u.oracle_reduce(d, xf)
    assert [k[0], v[0]] == g["argmin"]


# cpp/tests/core/operators_host.cpp:134-172: truth table of argmin_op / argmax_op on
# a=(0,1.2) b=(0,3.4) c=(1,1.2), in both argument orders.  A two-element row plus
# `init` plays the two operands.
def _arg2(red, first, second):
    """fold of [first, second] where each is (key, value): keys are forced through
    init (key of `first`) and a one-element row whose index is the key of `second`."""
    kf, vf = first
    ks, vs = second
    row = np.full(ks + 1, np.nan, dtype=np.float32)  # NaN never wins, pads the index
    row[ks] = vs
    d = api.make_desc(api.F32, api.KVP_I32_F32, 1, ks + 1, main_op=api.MAIN_KVP,
                      reduce_op=red, init_i=kf, init_f=vf)
    k, v = u.oracle_reduce(d, row)
    return int(k[0]), float(np.float32(v[0]))


def test_arg_op_truth_table(oracle):
    g = GOLD["arg_op_truth_table"]
    pair = {n: (kv[0], np.float32(kv[1])) for n, kv in g["pairs"].items()}
    f = lambda kv: (kv[0], float(kv[1]))
    for red, table in [(api.RED_ARGMIN, g["argmin"]), (api.RED_ARGMAX, g["argmax"])]:
        for x, y, want in table:
            assert _arg2(red, pair[x], pair[y]) == f(pair[want]), (red, x, y)


# cpp/tests/stats/sum.cu:50-98,108-140: the reference's grid of constant matrices (Result) and
# of (3v, -vL, +vL) triples (Accuracy); the column sums must be rows * value.  Cases above a
# million elements run on the GPU only (tests/test_gpu_reference_stats.py).
def sum_case_matrix(npdt, rows, cols, value, large=None):
    """The reference's input for one SumInputs case, as a [rows, cols] array of npdt."""
    v = float(npdt(value))            # params.value is a T
    col = np.full(rows, v, dtype=np.float64)
    if large is not None:
        r = np.arange(rows)
        col[r % 3 == 2] = v * large
        col[(r % 3 == 1) & (r + 1 < rows)] = -v * large
        col[(r % 3 == 0) & (r + 2 < rows)] = 3.0 * v
    return np.repeat(col.astype(npdt)[:, None], cols, axis=1)


SUM_SMALL = [(k, c) for k in ("float", "double") for c in GOLD["stats_sum"][k] if c[1] * c[2] <= 10**6]


@pytest.mark.parametrize("kind,case", SUM_SMALL, ids=lambda x: str(x))
@pytest.mark.parametrize("accuracy", [False, True])
def test_sum_grid(oracle, kind, case, accuracy):
    g = GOLD["stats_sum"]
    tol, rows, cols, row_major, value = case
    npdt, dt = (np.float32, api.F32) if kind == "float" else (np.float64, api.F64)
    m = sum_case_matrix(npdt, rows, cols, value, g["large_factor"][kind] if accuracy else None)
    flat = np.ascontiguousarray(m.reshape(-1) if row_major else m.T.reshape(-1))
    d = api.make_desc(dt, dt, rows, cols, apply=api.ALONG_COLUMNS,
                      layout=api.ROW_MAJOR if row_major else api.COL_MAJOR)
    expected = np.full(cols, float(npdt(rows * float(npdt(value)))))
    eps = tol * (g["accuracy_tolerance_factor"] if accuracy else 1)
    # the typed implementation carries the reference's compensation term
    out = np.zeros(cols, dtype=npdt)
    u.oracle_typed(d, flat, out)
    assert u.approx_ok(out, expected, eps).all(), (out[:3], expected[:3])
    # the sequential fp64 oracle: exact on fp32 data to far below the tolerance
    if npdt == np.float32:
        assert u.approx_ok(u.oracle_reduce(d, flat), expected, 1e-6).all()


# cpp/tests/stats/stddev.cu:119-202: stddev of normal(mean, stddev) data within `tolerance` of
# the distribution's stddev, 0 for a single row, sqrt(vars) == stddev; the reference's RNG is not
# reproduced, numpy's normal stands in.  The 2^27-row constant cases run on the GPU only; their
# small-scale counterpart (constant data -> 0) is the last block.
@pytest.mark.parametrize("kind", ["float", "double"])
def test_stddev_grid(oracle, kind):
    npdt, dt = (np.float32, api.F32) if kind == "float" else (np.float64, api.F64)
    rng = np.random.default_rng(1234)
    for tol, mean, sd, rows, cols, sample, row_major in GOLD["stats_stddev"][kind]:
        if rows * cols > 10**6:
            rows = 4096  # same constant data, a size the CPU finishes at once
        m = (rng.normal(mean, sd, (rows, cols)) if sd > 0 else np.full((rows, cols), mean)).astype(npdt)
        flat = np.ascontiguousarray(m.reshape(-1) if row_major else m.T.reshape(-1))
        lay = api.ROW_MAJOR if row_major else api.COL_MAJOR
        mu = m.astype(np.float64).mean(axis=0)
        r = 1.0 / (rows - 1 if sample else rows)
        rm = r * rows if sample else 1.0
        ds = api.make_desc(dt, dt, rows, cols, layout=lay, apply=api.ALONG_COLUMNS,
                           main_op=api.MAIN_SQ, final_op=api.FIN_STDDEV_FROM_SUMSQ,
                           final_scalar=r, final_scalar2=rm)
        got = u.oracle_reduce(ds, flat, aux=mu)
        want = 0.0 if rows == 1 else sd
        assert u.approx_ok(got, np.full(cols, want), tol).all(), (rows, cols, got[:3])
        if rows > 1:
            assert np.allclose(got, m.astype(np.float64).std(axis=0, ddof=1 if sample else 0),
                               rtol=1e-9, atol=1e-7)
        ds.final_op = api.FIN_VAR_FROM_SUMSQ
        var = u.oracle_reduce(ds, flat, aux=mu)
        assert u.approx_ok(np.sqrt(var), got, tol).all()


# cpp/tests/stats/mean.cu:118-215: column means of normal(mean, stddev) data within `tolerance`
# of the mean, including half -> float and (rounded normals) int8 -> half.
@pytest.mark.parametrize("kind", ["float", "double", "half_to_float", "int8_to_half"])
def test_mean_grid(oracle, kind):
    in_np, in_dt, out_np, out_dt = {
        "float": (np.float32, api.F32, np.float32, api.F32),
        "double": (np.float64, api.F64, np.float64, api.F64),
        "half_to_float": (np.float16, api.F16, np.float32, api.F32),
        "int8_to_half": (np.int8, api.I8, np.float16, api.F16)}[kind]
    rng = np.random.default_rng(1234)
    for tol, mean, rows, cols, row_major, sd in GOLD["stats_mean"][kind]:
        if rows * cols > 10**7:
            continue  # GPU only
        x = rng.normal(mean, sd, (rows, cols))
        m = np.clip(np.rint(x), -128, 127).astype(np.int8) if in_np == np.int8 else x.astype(in_np)
        flat = np.ascontiguousarray(m.reshape(-1) if row_major else m.T.reshape(-1))
        ratio = float(out_np(1) / out_np(rows))   # stats/detail/mean.cuh:22
        d = api.make_desc(in_dt, out_dt, rows, cols, apply=api.ALONG_COLUMNS,
                          layout=api.ROW_MAJOR if row_major else api.COL_MAJOR,
                          final_op=api.FIN_MUL_CONST, final_scalar=ratio)
        got = u.oracle_reduce(d, flat)
        if in_np == np.int8:
            assert np.all(np.abs(got - mean) <= tol)            # ASSERT_NEAR
        else:
            assert u.approx_ok(got, np.full(cols, float(in_np(mean))), tol).all()
        assert np.allclose(got, m.astype(np.float64).sum(axis=0) * ratio, rtol=1e-12)
        out = np.zeros(cols, dtype=out_np)
        u.oracle_typed(d, flat, out)
        assert np.allclose(out.astype(np.float64), got, rtol=2e-3 if out_np == np.float16 else 1e-5)


# core/math.hpp:375-397,517-533: the device max / min ignore NaN (fmax / fmin); a row of NaN
# only returns `init`.  numpy's nanmax / nanmin are the independent statement of that rule.
@pytest.mark.parametrize("layout,apply", itertools.product([api.ROW_MAJOR, api.COL_MAJOR],
                                                           [api.ALONG_ROWS, api.ALONG_COLUMNS]))
def test_max_min_ignore_nan(oracle, layout, apply):
    rng = np.random.default_rng(17)
    rows, cols = 23, 31
    m = rng.standard_normal((rows, cols)).astype(np.float32)
    m[rng.random((rows, cols)) < 0.2] = np.nan
    m[4, :] = np.nan
    m[:, 7] = np.nan
    flat = np.ascontiguousarray(m.reshape(-1) if layout == api.ROW_MAJOR else m.T.reshape(-1))
    ax = 1 if apply == api.ALONG_ROWS else 0
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)
        cases = [(api.MAIN_IDENTITY, api.RED_MAX, -np.inf, np.nanmax(m, axis=ax)),
                 (api.MAIN_IDENTITY, api.RED_MIN, np.inf, np.nanmin(m, axis=ax)),
                 (api.MAIN_ABS, api.RED_MAX, 0.0, np.nanmax(np.abs(m), axis=ax))]   # Linf norm
    for main, red, init, want in cases:
        want = np.where(np.isnan(want), init, want).astype(np.float64)
        d = api.make_desc(api.F32, api.F32, rows, cols, layout=layout, apply=apply, main_op=main,
                          reduce_op=red, init_f=init)
        assert np.array_equal(u.oracle_reduce(d, flat), want), (main, red)
        out = np.zeros(len(want), dtype=np.float32)
        assert np.array_equal(u.oracle_typed(d, flat, out).astype(np.float64), want), (main, red)


# cpp/tests/linalg/map_then_reduce.cu:140-169
def test_map_reduce_planted(oracle):
    g = GOLD["map_reduce_planted"]
    rng = np.random.default_rng(1234)
    x = rng.uniform(g["lo"], g["hi"], g["len"]).astype(np.float32)
    for pos, val in g["planted"].items():
        x[int(pos)] = val
    d = api.make_desc(api.F32, api.F32, 1, x.size, reduce_op=api.RED_MIN, init_f=np.inf)
    assert u.oracle_reduce(d, x).tolist() == [g["min"]]
    d = api.make_desc(api.F32, api.F32, 1, x.size, reduce_op=api.RED_MAX, init_f=-np.inf)
    assert u.oracle_reduce(d, x).tolist() == [g["max"]]


# What the mathematics fixes: numpy's own reductions on a non-square random matrix for
# all four layout x axis combinations (a swapped stride or axis changes the answer).
@pytest.mark.parametrize("layout,apply", itertools.product([api.ROW_MAJOR, api.COL_MAJOR],
                                                           [api.ALONG_ROWS, api.ALONG_COLUMNS]))
def test_against_numpy_closed_forms(oracle, layout, apply):
    rng = np.random.default_rng(7)
    rows, cols = 13, 29
    m = rng.standard_normal((rows, cols))
    flat = m.reshape(-1) if layout == api.ROW_MAJOR else m.T.reshape(-1)
    flat = np.ascontiguousarray(flat)
    ax = 1 if apply == api.ALONG_ROWS else 0
    cases = [
        (api.MAIN_IDENTITY, api.RED_ADD, api.FIN_IDENTITY, 0.0, m.sum(axis=ax)),
        (api.MAIN_SQ, api.RED_ADD, api.FIN_SQRT, 0.0, np.linalg.norm(m, axis=ax)),
        (api.MAIN_ABS, api.RED_ADD, api.FIN_IDENTITY, 0.0, np.abs(m).sum(axis=ax)),
        (api.MAIN_ABS, api.RED_MAX, api.FIN_IDENTITY, 0.0, np.abs(m).max(axis=ax)),
        (api.MAIN_IDENTITY, api.RED_MIN, api.FIN_IDENTITY, np.inf, m.min(axis=ax)),
        (api.MAIN_NZ, api.RED_ADD, api.FIN_IDENTITY, 0.0, (m != 0).sum(axis=ax)),
    ]
    for main, red, fin, init, want in cases:
        d = api.make_desc(api.F64, api.F64, rows, cols, layout=layout, apply=apply, main_op=main,
                          reduce_op=red, final_op=fin, init_f=init)
        got = u.oracle_reduce(d, flat)
        assert np.allclose(got, want, rtol=1e-13, atol=0), (main, red)
        out = np.zeros(len(want))
        assert np.allclose(u.oracle_typed(d, flat, out), want, rtol=1e-13, atol=0)
    # mean / population and sample stddev against numpy
    n = m.shape[1 - ax] if False else (cols if ax == 1 else rows)
    d = api.make_desc(api.F64, api.F64, rows, cols, layout=layout, apply=apply,
                      final_op=api.FIN_MUL_CONST, final_scalar=1.0 / n)
    mu = u.oracle_reduce(d, flat)
    assert np.allclose(mu, m.mean(axis=ax), rtol=1e-13)
    for sample in (False, True):
        r = 1.0 / (n - 1 if sample else n)
        rm = r * n if sample else 1.0
        d = api.make_desc(api.F64, api.F64, rows, cols, layout=layout, apply=apply,
                          main_op=api.MAIN_SQ, final_op=api.FIN_STDDEV_FROM_SUMSQ,
                          final_scalar=r, final_scalar2=rm)
        sd = u.oracle_reduce(d, flat, aux=mu)
        assert np.allclose(sd, m.std(axis=ax, ddof=1 if sample else 0), rtol=1e-10)
    # arg reductions against numpy's first-extremum rule, with planted ties
    mt = m.copy()
    mt[:, 5] = mt[:, 20] = 50.0
    mt[3, :] = mt[9, :] = -50.0
    flat_t = np.ascontiguousarray(mt.reshape(-1) if layout == api.ROW_MAJOR else mt.T.reshape(-1))
    d = api.make_desc(api.F64, api.KVP_I64_F64, rows, cols, layout=layout, apply=apply,
                      main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, init_f=-np.inf)
    k, v = u.oracle_reduce(d, flat_t)
    assert np.array_equal(k, np.argmax(mt, axis=ax)) and np.array_equal(v, mt.max(axis=ax))
    d.reduce_op = api.RED_ARGMIN
    d.init.f = np.inf
    k, v = u.oracle_reduce(d, flat_t)
    assert np.array_equal(k, np.argmin(mt, axis=ax)) and np.array_equal(v, mt.min(axis=ax))


# inplace: dots = final(red(dots_old, acc)) -- tests/linalg/reduce.cuh:42-46
def test_inplace_and_init(oracle):
    x = np.arange(12, dtype=np.float64)
    d = api.make_desc(api.F64, api.F64, 3, 4, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT,
                      inplace=True)
    old = np.array([1.0, 2.0, 3.0])
    want = np.sqrt(old + (x.reshape(3, 4) ** 2).sum(axis=1))
    assert np.allclose(u.oracle_reduce(d, x, old=old), want, rtol=1e-15)
    out = old.copy()
    assert np.allclose(u.oracle_typed(d, x, out), want, rtol=1e-15)
    di = api.make_desc(api.I32, api.I64, 3, 4, init_i=0, final_op=api.FIN_MUL_CONST,
                       final_scalar=3)
    xi = np.arange(12, dtype=np.int32)
    assert u.oracle_reduce(di, xi).tolist() == (3 * xi.reshape(3, 4).sum(axis=1)).tolist()


# integers: exact against numpy in int64, all integer input types
@pytest.mark.parametrize("dt,npdt", [(api.I8, np.int8), (api.U8, np.uint8), (api.I32, np.int32),
                                     (api.I64, np.int64)])
def test_integer_sums_exact(oracle, dt, npdt):
    rng = np.random.default_rng(11)
    info = np.iinfo(npdt)
    lo, hi = max(info.min, -2**40), min(info.max, 2**40)
    m = rng.integers(lo, hi, (37, 1001), dtype=npdt)
    for main, f in [(api.MAIN_IDENTITY, lambda a: a), (api.MAIN_ABS, np.abs)]:
        d = api.make_desc(dt, api.I64, 37, 1001, main_op=main)
        want = f(m.astype(np.int64)).sum(axis=1)
        assert np.array_equal(u.oracle_reduce(d, m.reshape(-1)), want)
        out = np.zeros(37, dtype=np.int64)
        assert np.array_equal(u.oracle_typed(d, m.reshape(-1), out), want)


# storage conversions against numpy's float16 and a bit-level bf16 rule
def test_storage_conversions(oracle):
    import ctypes as C
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(4000).astype(np.float32) * 100,
                        np.array([0.0, -0.0, 1e-8, -1e-8, 65504, 70000, 6e-8, np.inf, -np.inf],
                                 dtype=np.float32)])
    h = np.empty(x.size, dtype=np.uint16)
    oracle.orc_f32_to_f16(x.ctypes.data, h.ctypes.data, x.size)
    assert np.array_equal(h, x.astype(np.float16).view(np.uint16))
    back = np.empty(x.size, dtype=np.float32)
    oracle.orc_f16_to_f32(h.ctypes.data, back.ctypes.data, x.size)
    assert np.array_equal(back, h.view(np.float16).astype(np.float32))
    allh = np.arange(65536, dtype=np.uint16)
    backall = np.empty(65536, dtype=np.float32)
    oracle.orc_f16_to_f32(allh.ctypes.data, backall.ctypes.data, 65536)
    ref = allh.view(np.float16).astype(np.float32)
    assert np.array_equal(backall.view(np.uint32), ref.view(np.uint32))
    # bf16 against torch's conversion (an independent implementation): random bit patterns of
    # every exponent, and exact ties (the low 16 bits are 0x8000), which must go to even
    import torch
    bits = rng.integers(0, 2**32, 4_000_000, dtype=np.uint64).astype(np.uint32)
    ties = (rng.integers(0, 2**16, 100_000, dtype=np.uint64).astype(np.uint32) << 16) | 0x8000
    xb = np.concatenate([bits, ties, x.view(np.uint32)]).view(np.float32)
    xb = xb[~np.isnan(xb)]
    b = u.to_bf16(xb)
    want = torch.from_numpy(xb).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(b, want)
    assert np.array_equal(u.from_bf16(b).view(np.uint32),
                          torch.from_numpy(b.view(np.int16)).view(torch.bfloat16).float().numpy().view(np.uint32))
    nan = u.to_bf16(np.array([np.nan], dtype=np.float32))
    assert np.isnan(u.from_bf16(nan)[0])


# the OpenMP implementation agrees with the sequential oracle on the benchmark's
# kinds of input, to the build's floating tolerance / exactly for integers and keys
def test_typed_matches_sequential(oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal(3000 * 128).astype(np.float32)
    d = api.make_desc(api.F32, api.F32, 3000, 128, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
    out = np.zeros(3000, dtype=np.float32)
    assert u.fp_close(u.oracle_typed(d, x, out), u.oracle_reduce(d, x)).all()
    x = (3 + 2 * rng.standard_normal(40000 * 64)).astype(np.float32)
    d = api.make_desc(api.F32, api.F32, 40000, 64, apply=api.ALONG_COLUMNS,
                      final_op=api.FIN_MUL_CONST, final_scalar=1.0 / 40000)
    out = np.zeros(64, dtype=np.float32)
    assert u.fp_close(u.oracle_typed(d, x, out), u.oracle_reduce(d, x)).all()
    m = rng.standard_normal((50, 32000)).astype(np.float32)
    m[:, 100] = m[:, 31000] = 7.0
    d = api.make_desc(api.F32, api.KVP_I32_F32, 50, 32000, main_op=api.MAIN_KVP,
                      reduce_op=api.RED_ARGMAX, init_f=-np.inf)
    out = np.zeros(50, dtype=u.KVP_NP[api.KVP_I32_F32])
    u.oracle_typed(d, m.reshape(-1), out)
    k, v = u.oracle_reduce(d, m.reshape(-1))
    assert np.array_equal(out["key"], k) and (k == 100).all()
    assert np.array_equal(out["value"].astype(np.float64), v)
    xb = u.to_bf16(rng.uniform(-1, 1, 2 * 100000).astype(np.float32))
    d = api.make_desc(api.BF16, api.F32, 2, 100000)
    out = np.zeros(2, dtype=np.float32)
    assert u.fp_close(u.oracle_typed(d, xb, out), u.oracle_reduce(d, xb)).all()


# row normalisation against numpy: x / ||x|| per row for the three norms, rows below
# eps keep their previous contents (cpp/include/raft/linalg/detail/normalize.cuh:52-56)
def test_row_normalize_against_numpy(oracle):
    import ctypes as C
    rng = np.random.default_rng(21)
    rows, cols = 17, 29
    m = rng.standard_normal((rows, cols))
    m[5] = 0.0
    cases = [(api.MAIN_ABS, api.RED_ADD, api.FIN_IDENTITY, np.abs(m).sum(axis=1)),
             (api.MAIN_SQ, api.RED_ADD, api.FIN_SQRT, np.linalg.norm(m, axis=1)),
             (api.MAIN_ABS, api.RED_MAX, api.FIN_IDENTITY, np.abs(m).max(axis=1))]
    for main, red, fin, norms in cases:
        d = api.make_desc(api.F64, api.F64, rows, cols, main_op=main, reduce_op=red, final_op=fin)
        out = np.full(rows * cols, -1.0)
        rc = oracle.orc_row_normalize(C.byref(d), m.ctypes.data, out.ctypes.data, 1e-8)
        assert rc == 0
        out = out.reshape(rows, cols)
        want = np.where(norms[:, None] > 1e-8, m / np.where(norms > 0, norms, 1.0)[:, None], -1.0)
        assert np.allclose(out, want, rtol=1e-14, atol=0)
        assert (out[5] == -1.0).all()
    # A NaN norm is not <= eps (linalg/detail/normalize.cuh:52,120): the row is written, as NaN.
    # Sums turn NaN with one NaN element; the NaN-ignoring max does not, so that row is divided
    # by the largest of its other elements.
    mn = m.copy()
    mn[2, 11] = np.nan
    for main, red, fin, norms in cases:
        d = api.make_desc(api.F64, api.F64, rows, cols, main_op=main, reduce_op=red, final_op=fin)
        out = np.full(rows * cols, -1.0)
        assert oracle.orc_row_normalize(C.byref(d), mn.ctypes.data, out.ctypes.data, 1e-8) == 0
        out = out.reshape(rows, cols)
        if red == api.RED_ADD:
            assert np.isnan(out[2]).all()
        else:
            want2 = mn[2] / np.nanmax(np.abs(mn[2]))
            assert np.isnan(out[2, 11]) and np.allclose(np.delete(out[2], 11), np.delete(want2, 11), rtol=1e-14)
        assert np.allclose(out[3], m[3] / norms[3], rtol=1e-14)


# ---- one-pass mean and variance -------------------------------------------------------
# orc_meanvar restates the reference's running merge; numpy's two-pass mean / var fix
# what it must produce.  A wrong merge weight, a missing cross term or N instead of N-1
# each fail the 1e-12 bar; the reference's own statistical bound on normal data
# (cpp/tests/stats/meanvar.cu:27-33,127-150) is checked beside it.
@pytest.mark.parametrize("npdt,dt", [(np.float32, api.F32), (np.float64, api.F64)])
@pytest.mark.parametrize("layout", [api.ROW_MAJOR, api.COL_MAJOR])
@pytest.mark.parametrize("sample", [False, True])
def test_meanvar_against_numpy(oracle, npdt, dt, layout, sample):
    rng = np.random.default_rng(1234)
    for rows, cols, mu, sd in [(1024, 32, 1.0, 2.0), (700, 13, -1.0, 2.0), (1, 5, 3.0, 1.0),
                               (2, 3, 1e4, 1e-2), (257, 1, 0.0, 1.0)]:
        m = rng.normal(mu, sd, (rows, cols)).astype(npdt)
        stored = np.ascontiguousarray(m if layout == api.ROW_MAJOR else m.T)
        mean = np.zeros(cols)
        var = np.zeros(cols)
        rc = oracle.orc_meanvar(dt, layout, rows, cols, int(sample), stored.ctypes.data,
                                mean.ctypes.data, var.ctypes.data)
        assert rc == 0
        m64 = m.astype(np.float64)
        exp_mean = m64.mean(axis=0)
        exp_var = m64.var(axis=0, ddof=1 if sample and rows > 1 else 0)
        np.testing.assert_allclose(mean, exp_mean, rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(var, exp_var, rtol=1e-9, atol=1e-12)
        if rows >= 700 and sd == 2.0:
            assert np.all(np.abs(mean - mu) <= 6 * sd / np.sqrt(rows))
            assert np.all(np.abs(var - sd * sd) <= 6 * sd * sd * np.sqrt(2.0 / (rows - 1)))


# ---- covariance ------------------------------------------------------------------------
# orc_cov restates "mean-centre in the data's type, then alpha * X^T X".  The reference's
# own known answer (cpp/tests/stats/cov.cu:88-100,163-177) and numpy.cov fix what it must
# produce: ddof distinguishes N from N - 1, the non-square shapes and both layouts catch a
# transposed operand or a wrong stride, a mean far from zero catches a dropped centring.
def _orc_cov(oracle, dt, layout, rows, cols, sample, stored, mu, want_centered=False):
    covar = np.zeros((cols, cols))
    cen = np.zeros_like(stored) if want_centered else None
    rc = oracle.orc_cov(dt, layout, rows, cols, int(sample), stored.ctypes.data,
                        mu.ctypes.data if mu is not None else None, covar.ctypes.data,
                        cen.ctypes.data if cen is not None else None)
    assert rc == 0
    return covar, cen


@pytest.mark.parametrize("npdt,dt", [(np.float32, api.F32), (np.float64, api.F64)])
def test_cov_known_answer_fixture(oracle, npdt, dt):
    k = GOLD["stats_cov"]["known_answer"]
    data = np.array(k["data"], dtype=npdt)  # column-major 3 x 2
    m = data.reshape(k["cols"], k["rows"]).T
    mu = m.mean(axis=0).astype(npdt)
    covar, _ = _orc_cov(oracle, dt, api.COL_MAJOR, k["rows"], k["cols"], k["sample"], data, mu)
    tol = 2 * GOLD["stats_cov"]["cases"][0][0]
    exp = np.array(k["covar"]).reshape(2, 2)
    assert np.all(np.abs(covar - exp) <= tol * np.maximum(1.0, np.abs(exp)))
    np.testing.assert_allclose(covar, np.cov(m.astype(np.float64), rowvar=False, ddof=1), rtol=1e-6)


@pytest.mark.parametrize("npdt,dt,rtol", [(np.float32, api.F32, 2e-6), (np.float64, api.F64, 1e-12)])
@pytest.mark.parametrize("layout", [api.ROW_MAJOR, api.COL_MAJOR])
@pytest.mark.parametrize("sample", [False, True])
def test_cov_against_numpy(oracle, npdt, dt, rtol, layout, sample):
    rng = np.random.default_rng(99)
    for rows, cols, mean in [(1000, 7, 3.0), (257, 33, -1.0), (64, 70, 100.0), (2, 3, 0.5)]:
        m = (rng.normal(mean, 2.0, (rows, cols)) * rng.uniform(0.5, 2.0, cols)).astype(npdt)
        stored = np.ascontiguousarray(m if layout == api.ROW_MAJOR else m.T).reshape(-1)
        mu = m.astype(np.float64).mean(axis=0).astype(npdt)
        covar, cen = _orc_cov(oracle, dt, layout, rows, cols, sample, stored, mu, True)
        exp = np.cov(m.astype(np.float64), rowvar=False, ddof=1 if sample else 0)
        scale = np.sqrt(np.outer(np.diag(exp), np.diag(exp)))
        # the data is centred in its own type around a mean rounded to that type
        assert np.all(np.abs(covar - exp) <= rtol * scale * max(1.0, abs(mean))), (rows, cols)
        assert np.array_equal(covar, covar.T)
        # what the reference leaves in `data`
        cen_m = cen.reshape(rows, cols) if layout == api.ROW_MAJOR else cen.reshape(cols, rows).T
        assert np.array_equal(cen_m, (m - mu[None, :]).astype(npdt))
        # mu == NULL: the data is taken as centred
        c2, _ = _orc_cov(oracle, dt, layout, rows, cols, sample, cen, None)
        assert np.array_equal(c2, covar)
