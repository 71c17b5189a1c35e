"""Row normalisation (rmi_row_normalize) on the GPU against the fp64 oracle: the shape
grid of the reference's test (cpp/tests/linalg/normalize.cu:111-135), long rows, half
types, rows below eps left untouched, in-place use."""
import ctypes as C
import itertools

import numpy as np
import pytest

from raft_amd import _capi as api
from tests import _util as u

pytestmark = pytest.mark.gpu

NORMS = {
    "l1": (api.MAIN_ABS, api.RED_ADD, api.FIN_IDENTITY),
    "l2": (api.MAIN_SQ, api.RED_ADD, api.FIN_SQRT),
    "linf": (api.MAIN_ABS, api.RED_MAX, api.FIN_IDENTITY),
}


def _oracle(desc, data, prev, eps):
    out = np.ascontiguousarray(prev, dtype=np.float64).copy()
    rc = u.load_oracle().orc_row_normalize(C.byref(desc), data.ctypes.data, out.ctypes.data, eps)
    assert rc == 0
    return out


def _gpu(desc, data, prev_raw, eps, inplace=False):
    import torch
    from raft_amd import device as dev
    x = torch.from_numpy(data.view(np.uint8).reshape(-1)).cuda()
    o = x if inplace else torch.from_numpy(prev_raw.view(np.uint8).reshape(-1).copy()).cuda()
    rc = api.load().rmi_row_normalize(C.byref(desc), x.data_ptr(), o.data_ptr(), eps,
                                      dev.current_stream_ptr())
    assert rc == 0, api.status_string(rc)
    torch.cuda.synchronize()
    return o.cpu().numpy().view(data.dtype).copy()


def _as_f64(dt, raw):
    return u.from_bf16(raw).astype(np.float64) if dt == api.BF16 else raw.astype(np.float64)


@pytest.mark.parametrize("dt,npdt,tol", [(api.F32, np.float32, 1e-5), (api.F64, np.float64, 1e-8)])
@pytest.mark.parametrize("norm", list(NORMS))
@pytest.mark.parametrize("rows,cols", itertools.product([11, 101, 12345],
                                                        [2, 3, 7, 12, 33, 125, 254]))
def test_reference_grid(gpu, dt, npdt, tol, norm, rows, cols):
    rng = np.random.default_rng(1234)
    data = rng.uniform(-10, 10, rows * cols).astype(npdt)
    main, red, fin = NORMS[norm]
    d = api.make_desc(dt, dt, rows, cols, main_op=main, reduce_op=red, final_op=fin)
    prev = np.full(rows * cols, 7.0, dtype=npdt)
    got = _gpu(d, data, prev, 1e-8)
    exp = _oracle(d, data, prev, 1e-8)
    assert u.approx_ok(got, exp, tol).all(), u.worst_rel(got, exp)


@pytest.mark.parametrize("rows,cols", [(37, 1024), (9, 5000), (5, 70001), (3, 1 << 18), (2000, 1000),
                                       (21, 4001), (13, 16003), (7, 30000), (6, 60002), (40, 65536)])
@pytest.mark.parametrize("norm", ["l1", "l2", "linf"])
def test_long_rows(gpu, rows, cols, norm):
    rng = np.random.default_rng(cols)
    data = rng.standard_normal(rows * cols).astype(np.float32)
    main, red, fin = NORMS[norm]
    d = api.make_desc(api.F32, api.F32, rows, cols, main_op=main, reduce_op=red, final_op=fin)
    prev = np.zeros(rows * cols, dtype=np.float32)
    got = _gpu(d, data, prev, 1e-8)
    exp = _oracle(d, data, prev, 1e-8)
    assert u.approx_ok(got, exp, 1e-5).all(), u.worst_rel(got, exp)
    if norm == "l2":  # unit rows
        n = np.linalg.norm(got.reshape(rows, cols).astype(np.float64), axis=1)
        assert np.allclose(n, 1.0, atol=1e-5)


# Rows whose lane-load count is not a power of two take one lane per lane-load (3..32 and
# 54..63 lane-loads, whole rows per wave step) or three loads per lane; row counts around
# one wave's and one workgroup's share.
@pytest.mark.parametrize("cols", [10, 20, 21, 45, 50, 67, 100, 127, 129, 190, 200, 222, 250, 255, 300])
@pytest.mark.parametrize("rows", [1, 5, 29, 257, 4099])
def test_lane_counts(gpu, rows, cols):
    rng = np.random.default_rng(rows * 1000 + cols)
    data = rng.uniform(-3, 3, rows * cols).astype(np.float32)
    d = api.make_desc(api.F32, api.F32, rows, cols, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
    prev = np.full(rows * cols, 9.0, dtype=np.float32)
    got = _gpu(d, data, prev, 1e-8)
    exp = _oracle(d, data, prev, 1e-8)
    assert u.approx_ok(got, exp, 1e-5).all(), u.worst_rel(got, exp)


@pytest.mark.parametrize("dt", [api.F16, api.BF16])
@pytest.mark.parametrize("rows,cols", [(100, 64), (1000, 100), (33, 7), (7, 9000), (500, 33), (301, 108),
                                       (64, 450)])
def test_half_types(gpu, dt, rows, cols):
    rng = np.random.default_rng(3)
    f = rng.uniform(-4, 4, rows * cols).astype(np.float32)
    data = f.astype(np.float16) if dt == api.F16 else u.to_bf16(f)
    d = api.make_desc(dt, dt, rows, cols, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
    prev = np.zeros(rows * cols, dtype=data.dtype)
    raw = _gpu(d, data, prev, 1e-8)
    exp = _oracle(d, data, _as_f64(dt, prev), 1e-8)
    # one rounding to 16 bits of x * (1 / norm) in fp32: the rounded oracle value or its neighbour
    assert u.ulp16_ok(dt, raw, exp).all(), u.worst_rel(_as_f64(dt, raw), exp)


def test_rows_below_eps_are_left_untouched(gpu):
    rows, cols = 64, 96
    rng = np.random.default_rng(8)
    m = rng.standard_normal((rows, cols)).astype(np.float32)
    m[::4] = 0.0          # norm 0
    m[1::8] *= 1e-12      # norm far below eps
    d = api.make_desc(api.F32, api.F32, rows, cols, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
    prev = np.full(rows * cols, -3.0, dtype=np.float32)
    got = _gpu(d, m.reshape(-1), prev, 1e-6).reshape(rows, cols)
    exp = _oracle(d, m.reshape(-1), prev, 1e-6).reshape(rows, cols)
    assert (got[::4] == -3.0).all() and (got[1::8] == -3.0).all()
    assert u.approx_ok(got, exp, 1e-5).all()


@pytest.mark.parametrize("rows,cols", [(1000, 128), (50, 33), (4, 20000)])
def test_in_place(gpu, rows, cols):
    rng = np.random.default_rng(rows)
    data = rng.standard_normal(rows * cols).astype(np.float32)
    d = api.make_desc(api.F32, api.F32, rows, cols, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
    got = _gpu(d, data, None, 1e-8, inplace=True)
    exp = _oracle(d, data, data, 1e-8)
    assert u.approx_ok(got, exp, 1e-5).all(), u.worst_rel(got, exp)


# Rows too long for a team's registers (more than 16384 lane-loads) are swept twice, the second
# time re-reading the row while other waves already store: in place, the overlapping last
# vector of a row with tail elements must not pick up values another wave has scaled already.
# Lengths one past a multiple of 64 lane-loads put that vector's two owners in different waves.
@pytest.mark.parametrize("dt,cols", [(api.F32, 65537), (api.F32, 70145), (api.F32, 131073),
                                     (api.F32, 65536 + 256 * 4 + 3), (api.F64, 32769 + 2 * 64),
                                     (api.F16, 131073), (api.BF16, 131079), (api.F16, 140003)])
@pytest.mark.parametrize("norm", ["l2", "linf"])
def test_in_place_swept_rows(gpu, dt, cols, norm):
    rows = 6
    rng = np.random.default_rng(cols)
    f = rng.uniform(-4, 4, rows * cols)
    if dt == api.BF16:
        data = u.to_bf16(f.astype(np.float32))
    else:
        data = f.astype({api.F32: np.float32, api.F64: np.float64, api.F16: np.float16}[dt])
    main, red, fin = NORMS[norm]
    d = api.make_desc(dt, dt, rows, cols, main_op=main, reduce_op=red, final_op=fin)
    exp = _oracle(d, data, _as_f64(dt, data), 1e-8)
    for inplace in (True, False):
        raw = _gpu(d, data.copy(), np.zeros_like(data), 1e-8, inplace=inplace)
        if dt in (api.F16, api.BF16):
            ok = u.ulp16_ok(dt, raw, exp)
        else:
            ok = u.approx_ok(raw, exp, 1e-5 if dt == api.F32 else 1e-12)
        assert ok.all(), (inplace, np.flatnonzero(~ok)[:8] % cols)


# A row whose norm is NaN is not "<= eps" (linalg/detail/normalize.cuh:52,120): it is written,
# as NaN, not skipped.  Sums turn NaN with one NaN element; the NaN-ignoring max does not.
# Row lengths cover the wave kernels (power-of-two and any lane count), the team kernel and the
# two-sweep kernel.
@pytest.mark.parametrize("cols", [7, 33, 128, 1000, 5000, 70001])
@pytest.mark.parametrize("norm", ["l1", "l2", "linf"])
def test_nan_rows_are_written(gpu, cols, norm):
    rows = 9
    rng = np.random.default_rng(cols)
    m = rng.standard_normal((rows, cols)).astype(np.float32)
    m[2, cols // 3] = np.nan
    m[5, cols - 1] = np.nan
    main, red, fin = NORMS[norm]
    d = api.make_desc(api.F32, api.F32, rows, cols, main_op=main, reduce_op=red, final_op=fin)
    prev = np.full(rows * cols, -3.0, dtype=np.float32)
    got = _gpu(d, m.reshape(-1), prev, 1e-8).reshape(rows, cols)
    exp = _oracle(d, m.reshape(-1), prev, 1e-8).reshape(rows, cols)
    assert u.approx_ok(got, exp, 1e-5).all()
    if red == api.RED_ADD:
        assert np.isnan(got[2]).all() and np.isnan(got[5]).all()
    else:
        assert np.isnan(got[2]).sum() == 1 and np.isnan(got[5]).sum() == 1
    assert not np.isnan(got[[0, 1, 3, 4, 6, 7, 8]]).any() and not (got == -3.0).any()


# fp32 and fp64 rows are divided element by element in the reference (in / norm, a correctly
# rounded IEEE division).  The kernels compute the same quotient from one reciprocal and a
# residual correction; with the Linf norm the divisor is one of the row's own elements, so
# numpy's division in the same type gives the expected bits.  Rows scaled to 1e+-35 have a
# divisor outside the range where the shortcut is exact and take the division itself.
@pytest.mark.parametrize("dt,npdt", [(api.F32, np.float32), (api.F64, np.float64)])
@pytest.mark.parametrize("cols", [8, 100, 128, 1024, 5000, 70001])
def test_quotients_are_correctly_rounded(gpu, dt, npdt, cols):
    rows = 40
    rng = np.random.default_rng(cols)
    m = rng.standard_normal((rows, cols)) * np.exp(rng.uniform(-3, 3, (rows, cols)))
    m *= np.exp(rng.uniform(-20, 20, (rows, 1)))
    m[5] *= 1e35 / np.abs(m[5]).max()
    m[6] *= 1e-35 / np.abs(m[6]).max()
    m = m.astype(npdt)
    main, red, fin = NORMS["linf"]
    d = api.make_desc(dt, dt, rows, cols, main_op=main, reduce_op=red, final_op=fin)
    got = _gpu(d, m.reshape(-1), np.zeros(rows * cols, dtype=npdt), 0.0).reshape(rows, cols)
    want = m / np.abs(m).max(axis=1, keepdims=True)
    assert want.dtype == npdt
    assert np.array_equal(got, want), np.argwhere(got != want)[:5]


# Elements far below their row's norm: the residual of the reciprocal-and-correct quotient is
# not representable there (it falls below the subnormal spacing), so such elements must take
# the division itself.  Norm near 1, elements from 1e-30 down into the subnormals (fp32) and
# from 1e-290 down (fp64), held to numpy's division bit for bit.
@pytest.mark.parametrize("dt,npdt,lo_exp,hi_exp", [(api.F32, np.float32, -44.0, -30.0),
                                                    (api.F64, np.float64, -322.0, -290.0)])
def test_quotients_of_tiny_elements(gpu, dt, npdt, lo_exp, hi_exp):
    rows, cols = 64, 257
    rng = np.random.default_rng(5)
    m = (10.0 ** rng.uniform(lo_exp, hi_exp, (rows, cols)) * rng.choice([-1.0, 1.0], (rows, cols)))
    m[:, 0] = rng.uniform(0.05, 3000.0, rows)      # the row's L-inf norm
    m[:, 1] = rng.uniform(0.01, 0.04, rows) * m[:, 0]
    m = m.astype(npdt)
    main, red, fin = NORMS["linf"]
    d = api.make_desc(dt, dt, rows, cols, main_op=main, reduce_op=red, final_op=fin)
    got = _gpu(d, m.reshape(-1), np.zeros(rows * cols, dtype=npdt), 0.0).reshape(rows, cols)
    with np.errstate(under="ignore"):
        want = m / np.abs(m).max(axis=1, keepdims=True)
    assert want.dtype == npdt
    assert np.array_equal(got, want), (np.argwhere(got != want)[:5], got[got != want][:5],
                                       want[got != want][:5])


# Rows whose byte length is no multiple of 128 are normalised as a flat run of aligned
# 16-byte vectors (a vector holds parts of two rows; chunks of whole rows per workgroup).
# Row counts around the chunk sizes, every vector-to-row split, rows that must stay untouched
# (norm <= eps: their neighbours in the same vector are still written), NaN rows, outputs that
# start at every 16-byte offset into a 128-byte line, in place, and the few last rows that do
# not end on a 16-byte boundary (they take the row-wise kernels).
def _flat_case(dt, npdt, rows, cols, norm, in_off, out_off, inplace, seed):
    import torch
    from raft_amd import device as dev
    rng = np.random.default_rng(seed)
    m = rng.standard_normal((rows, cols)) * np.exp(rng.uniform(-2, 2, (rows, 1)))
    if rows > 3:
        m[rng.integers(0, rows, max(1, rows // 7))] = 0.0              # norm 0: untouched
        m[rng.integers(0, rows, max(1, rows // 11))] *= 1e-14           # norm below eps: untouched
    if rows > 5:
        m[rows // 2, cols // 3] = np.nan
    if dt == api.BF16:
        data = u.to_bf16(m.astype(np.float32).reshape(-1))
    else:
        data = m.astype(npdt).reshape(-1)
    es = data.dtype.itemsize
    main, red, fin = NORMS[norm]
    d = api.make_desc(dt, dt, rows, cols, main_op=main, reduce_op=red, final_op=fin)
    nbytes = rows * cols * es
    xbuf = torch.zeros(nbytes + 256, dtype=torch.uint8, device="cuda")
    xbuf[in_off:in_off + nbytes] = torch.from_numpy(data.view(np.uint8)).cuda()
    sentinel = np.full(rows * cols, 7.0, dtype=np.float32)
    prev = u.to_bf16(sentinel) if dt == api.BF16 else sentinel.astype(npdt)
    if inplace:
        obuf, out_off, prev_f64 = xbuf, in_off, _as_f64(dt, data)
    else:
        obuf = torch.zeros(nbytes + 256, dtype=torch.uint8, device="cuda")
        obuf[out_off:out_off + nbytes] = torch.from_numpy(prev.view(np.uint8)).cuda()
        prev_f64 = _as_f64(dt, prev)
    rc = api.load().rmi_row_normalize(C.byref(d), xbuf.data_ptr() + in_off, obuf.data_ptr() + out_off,
                                      1e-6, dev.current_stream_ptr())
    assert rc == 0, api.status_string(rc)
    torch.cuda.synchronize()
    got = obuf[out_off:out_off + nbytes].cpu().numpy().view(data.dtype).copy()
    assert (obuf[:out_off] == 0).all() and (obuf[out_off + nbytes:] == 0).all(), "wrote outside the matrix"
    exp = _oracle(d, data, prev_f64, 1e-6)
    if dt in (api.BF16, api.F16):
        ok = u.ulp16_ok(dt, got, exp)
    else:
        ok = u.approx_ok(got, exp, 1e-5 if dt == api.F32 else 1e-8)
    assert ok.all(), (rows, cols, norm, in_off, out_off, np.argwhere(~ok)[:4])
    if not inplace:  # untouched rows keep the output's old bits
        keep = exp.reshape(rows, cols) == 7.0
        assert (got.reshape(rows, cols)[keep] == prev.reshape(rows, cols)[keep]).all()


@pytest.mark.parametrize("dt,npdt,colset", [
    (api.F32, np.float32, (5, 9, 33, 100, 129, 250, 500, 1001)),
    (api.BF16, None, (9, 33, 100, 130, 1004)),
    (api.F16, np.float16, (12, 33, 500)),
    (api.F64, np.float64, (25, 33, 65, 250))])
def test_flat_rows(gpu, dt, npdt, colset):
    seed = 0
    for cols in colset:
        es = 2 if dt in (api.BF16, api.F16) else (4 if dt == api.F32 else 8)
        chunk = max(1, 16272 // (cols * es))
        for rows in sorted({1, 2, 7, 8, 9, 31, chunk - 1, chunk, chunk + 1, 2 * chunk + 3, 4099}):
            if rows < 1:
                continue
            seed += 1
            _flat_case(dt, npdt, rows, cols, ("l2", "l1", "linf")[seed % 3], 0, 0, seed % 4 == 0, seed)


@pytest.mark.parametrize("out_off", [16, 32, 48, 64, 80, 96, 112])
def test_flat_rows_at_line_offsets(gpu, out_off):
    for dt, npdt, cols in ((api.F32, np.float32, 129), (api.BF16, None, 33), (api.F64, np.float64, 33)):
        _flat_case(dt, npdt, 3001, cols, "l2", (out_off * 3) % 128, out_off, False, out_off + cols)
        _flat_case(dt, npdt, 3001, cols, "l2", out_off, out_off, True, out_off + cols + 1)


def test_full_size_embedding_shape(gpu):
    """1,000,000 x 128 fp32 (the shape of benchmark config 2): unit L2 rows, and the
    oracle on a slice."""
    import torch
    from raft_amd import device as dev
    rows, cols = 1000000, 128
    g = torch.Generator(device="cuda")
    g.manual_seed(2)
    x = torch.randn(rows * cols, generator=g, device="cuda")
    o = torch.empty_like(x)
    d = api.make_desc(api.F32, api.F32, rows, cols, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
    rc = api.load().rmi_row_normalize(C.byref(d), x.data_ptr(), o.data_ptr(), 1e-8,
                                      dev.current_stream_ptr())
    assert rc == 0
    n = torch.linalg.vector_norm(o.view(rows, cols).double(), dim=1)
    assert torch.allclose(n, torch.ones_like(n), atol=1e-6)
    ns = 5000
    sub = x[: ns * cols].cpu().numpy()
    ds = api.make_desc(api.F32, api.F32, ns, cols, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
    exp = _oracle(ds, sub, np.zeros(ns * cols), 1e-8)
    assert u.approx_ok(o[: ns * cols].cpu().numpy(), exp, 1e-5).all()


# Rows shorter than a 16-byte vector go through LDS (a chunk of whole rows as aligned vectors, a
# thread per row; 16-bit rows of an odd length are scaled vector by vector on the way out): row
# counts around a chunk, rows of norm 0 and below eps (untouched: their chunk is stored row by
# row), NaN, the three norms, in place, and starts off a 16-byte boundary (the other kernels).
@pytest.mark.gpu
@pytest.mark.parametrize("dt,npdt,colset", [
    (api.F32, np.float32, (2, 3)),
    (api.BF16, None, (2, 3, 4, 5, 6, 7)),
    (api.F16, np.float16, (3, 6)),
])
def test_rows_shorter_than_a_vector(gpu, dt, npdt, colset):
    es = 4 if dt == api.F32 else 2
    seed = 0
    for cols in colset:
        chunk = 16384 // (cols * es) // 16 * 16
        if es == 2 and cols % 2 == 1:
            chunk = min(chunk, 2048)
        for rows in sorted({1, 2, 17, chunk - 1, chunk, chunk + 1, 3 * chunk + 5}):
            for norm in NORMS:
                seed += 1
                _flat_case(dt, npdt, rows, cols, norm, 0, 0, seed % 3 == 0, seed)
            _flat_case(dt, npdt, rows, cols, "l2", 16, 48, False, seed + 1000)
            _flat_case(dt, npdt, rows, cols, "l2", es, 0, False, seed + 2000)      # off a 16-byte boundary
    # a chunk without any untouched row takes the whole-vector stores
    import torch
    from raft_amd import device as dev
    rng = np.random.default_rng(5)
    for cols in colset:
        rows = 50001
        m = rng.standard_normal((rows, cols)) + 3.0
        data = u.to_bf16(m.astype(np.float32).reshape(-1)) if dt == api.BF16 else m.astype(npdt).reshape(-1)
        d = api.make_desc(dt, dt, rows, cols, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
        x = torch.from_numpy(data.view(np.uint8)).cuda()
        o = torch.zeros_like(x)
        assert api.load().rmi_row_normalize(C.byref(d), x.data_ptr(), o.data_ptr(), 1e-6,
                                            dev.current_stream_ptr()) == 0
        torch.cuda.synchronize()
        got = o.cpu().numpy().view(data.dtype)
        exp = _oracle(d, data, np.zeros(rows * cols), 1e-6)
        ok = u.ulp16_ok(dt, got, exp) if dt in (api.BF16, api.F16) else u.approx_ok(got, exp, 1e-5)
        assert ok.all(), (cols, np.argwhere(~ok)[:4])


# Rows of 257 to 511 lane-loads stay on one wave with five to eight loads per lane: every load
# count, with and without tail elements, few rows and many, untouched and NaN rows, in place.
@pytest.mark.gpu
@pytest.mark.parametrize("dt,npdt,colset", [
    (api.F32, np.float32, (1025, 1028, 1281, 1300, 1537, 1791, 1793, 2040, 2043)),
    (api.BF16, None, (2049, 2056, 3000, 3585, 4081)),
    (api.F64, np.float64, (513, 640, 641, 1000, 1021)),
])
def test_rows_of_five_to_eight_loads_per_lane(gpu, dt, npdt, colset):
    seed = 0
    for cols in colset:
        for rows in (1, 5, 300):
            for norm in ("l2", "linf"):
                seed += 1
                _flat_case(dt, npdt, rows, cols, norm, 0, 0, seed % 3 == 0, seed)
        _flat_case(dt, npdt, 9, cols, "l1", 16, 64, False, seed + 500)
