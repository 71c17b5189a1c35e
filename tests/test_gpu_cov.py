"""Covariance (rmi_cov) on the GPU against the fp64 oracle: the reference's grid
(cpp/tests/stats/cov.cu:107-141) with its own checks, its 3 x 2 known answer, ragged shapes in
both layouts, the centred data the call leaves behind, error codes, and the 10,000,000 x 64
shape through size-independent properties.

Tolerance: an element of a Gram matrix is a dot product of two columns, so its rounding error
scales with the product of their norms: |got - oracle| <= 1e-5 * sqrt(C_ii * C_jj)."""
import ctypes as C

import numpy as np
import pytest

from raft_amd import _capi as api
from tests import _util as u

pytestmark = pytest.mark.gpu

NP = {api.F32: np.float32, api.F64: np.float64}
TOL = 1e-5
GOLD = u.golden()["stats_cov"]


def _oracle(dt, layout, rows, cols, sample, stored, mu):
    covar = np.zeros((cols, cols))
    cen = np.zeros_like(stored)
    rc = u.load_oracle().orc_cov(dt, layout, rows, cols, int(sample), stored.ctypes.data,
                                 mu.ctypes.data if mu is not None else None, covar.ctypes.data,
                                 cen.ctypes.data)
    assert rc == 0
    return covar, cen


def _gpu(dt, layout, rows, cols, sample, stored, mu, center):
    import torch
    from raft_amd import device as dev
    x = torch.from_numpy(stored.reshape(-1).copy()).cuda()
    m = torch.from_numpy(mu).cuda() if mu is not None else None
    out = torch.full((max(cols * cols, 1),), 77.0, dtype=x.dtype, device="cuda")
    dev.cov(dt, layout, rows, cols, sample, x, m, out, center=center)
    torch.cuda.synchronize()
    return out.cpu().numpy()[:cols * cols].reshape(cols, cols), x.cpu().numpy()


def _close(got, exp):
    d = np.sqrt(np.abs(np.diag(exp)))
    bound = TOL * np.outer(d, d) + 1e-300
    return np.abs(got.astype(np.float64) - exp) <= bound


def _check(dt, layout, rows, cols, sample, m, center, with_mu=True):
    stored = np.ascontiguousarray(m if layout == api.ROW_MAJOR else m.T).reshape(-1)
    mu = m.astype(np.float64).mean(axis=0).astype(NP[dt]) if with_mu else None
    exp, exp_cen = _oracle(dt, layout, rows, cols, sample, stored, mu)
    got, left = _gpu(dt, layout, rows, cols, sample, stored, mu, center)
    ok = _close(got, exp)
    assert ok.all(), (rows, cols, np.argwhere(~ok)[:4], got[~ok][:4], exp[~ok][:4])
    assert np.array_equal(got, got.T), "covar is written symmetric"
    # with RMI_COV_CENTER_DATA the call leaves x - mu (rounded once, like the reference's
    # meanCenter); without it the data is untouched
    want = exp_cen if (center and with_mu) else stored
    assert np.array_equal(left, want), (rows, cols, center)
    return got


# cpp/tests/stats/cov.cu:107-161: diagonal within 2 * tolerance of var * var (CompareApprox:
# |a - b| / max(|a|, |b|) <= eps), every element within 1e-5 of the oracle besides
@pytest.mark.parametrize("dt", [api.F32, api.F64])
@pytest.mark.parametrize("case", GOLD["cases"], ids=lambda c: f"{c[4]}c-s{int(c[5])}-rm{int(c[6])}")
def test_reference_grid(dt, case):
    tol, mean, sd, rows, cols, sample, row_major, stable = case
    assert stable  # the reference implements nothing else (stats/detail/cov.cuh:61-63)
    rng = np.random.default_rng(1234 + cols)
    m = rng.normal(mean, sd, (rows, cols)).astype(NP[dt])
    layout = api.ROW_MAJOR if row_major else api.COL_MAJOR
    got = _check(dt, layout, rows, cols, sample, m, center=True)
    diag = np.diag(got).astype(np.float64)
    want = sd * sd
    assert np.all(np.abs(diag - want) / np.maximum(np.abs(diag), want) <= 2 * tol)


# cpp/tests/stats/cov.cu:88-100,163-177
@pytest.mark.parametrize("dt", [api.F32, api.F64])
def test_known_answer(dt):
    k = GOLD["known_answer"]
    m = np.array(k["data"], dtype=NP[dt]).reshape(k["cols"], k["rows"]).T
    got = _check(dt, api.COL_MAJOR, k["rows"], k["cols"], k["sample"], m, center=True)
    exp = np.array(k["covar"]).reshape(2, 2)
    tol = 2 * GOLD["cases"][0][0]
    assert np.all(np.abs(got - exp) / np.maximum(np.abs(got), np.abs(exp)) <= tol)


SHAPES = [(1, 1), (2, 3), (3, 2), (15, 5), (16, 4), (17, 63), (31, 64), (33, 65), (100, 100),
          (257, 129), (1000, 130), (4099, 200), (513, 260), (64, 8), (5000, 66),
          (2, 32), (1000, 32), (1001, 32), (4096, 16), (40, 8), (96, 4)]

# Up to 32 columns and 4M elements or more: contracted as f D <= 64 columns, f = 64 // D rows side
# by side (row-major, the rows left over added separately) or the largest divisor of the row
# count up to that (col-major: pieces of whole columns)
NARROW = [(131072, 32), (131073, 32), (262144, 16), (262148, 16), (262146, 16), (524288, 8),
          (524292, 8), (1048576, 4), (1048592, 4), (1048577, 4),
          (1398101, 3), (1398120, 3), (4194304, 1), (4194305, 1), (2097153, 2), (838861, 5), (838860, 5),
          (600000, 7), (420001, 10), (349526, 12), (209716, 20), (209715, 20), (135301, 31), (190651, 22)]


@pytest.mark.parametrize("dt", [api.F32, api.F64])
@pytest.mark.parametrize("layout", [api.ROW_MAJOR, api.COL_MAJOR])
@pytest.mark.parametrize("center", [False, True])
def test_ragged_shapes(dt, layout, center):
    rng = np.random.default_rng(7 + dt + 10 * layout)
    for rows, cols in SHAPES:
        m = (rng.normal(3.0, 2.0, (rows, cols)) * rng.uniform(0.25, 4.0, cols)).astype(NP[dt])
        for sample in ((False, True) if rows > 1 else (False,)):
            _check(dt, layout, rows, cols, sample, m, center)


@pytest.mark.parametrize("dt", [api.F32, api.F64])
@pytest.mark.parametrize("layout", [api.ROW_MAJOR, api.COL_MAJOR])
@pytest.mark.parametrize("center", [False, True])
def test_narrow_matrices(dt, layout, center):
    rng = np.random.default_rng(21 + dt + 10 * layout)
    for rows, cols in NARROW:
        m = (rng.normal(1.0, 2.0, (rows, cols)) * rng.uniform(0.25, 4.0, cols)).astype(NP[dt])
        _check(dt, layout, rows, cols, rows % 2 == 0, m, center)


@pytest.mark.parametrize("layout", [api.ROW_MAJOR, api.COL_MAJOR])
@pytest.mark.parametrize("center", [False, True])
def test_one_block_few_units_per_wave(layout, center):
    """One whole block of 64 fp32 columns and so few rows that a wave gets 0 to 9 units of 32
    rows, with and without a ragged last unit: every entry and exit of the pipelined loop
    (prologue only, partial first trip, whole trips, the trip that ends on a dead unit)."""
    rng = np.random.default_rng(11 + layout)
    for rows in (32, 33, 64, 127, 128, 129, 160, 255, 256, 257, 384, 511, 512, 513, 640, 768,
                 1000, 1024, 1056, 1151, 1152, 1153, 1280, 2047, 2048, 2081):
        m = (rng.normal(-1.0, 3.0, (rows, 64)) * rng.uniform(0.5, 2.0, 64)).astype(np.float32)
        _check(api.F32, layout, rows, 64, True, m, center)
    for cols in (60, 32, 8):  # the same loops with masked columns
        m = rng.normal(0.5, 1.0, (1153, cols)).astype(np.float32)
        _check(api.F32, layout, 1153, cols, False, m, center)


@pytest.mark.parametrize("dt", [api.F32, api.F64])
@pytest.mark.parametrize("layout", [api.ROW_MAJOR, api.COL_MAJOR])
def test_without_mean_vector(dt, layout):
    """mu == NULL: the data is taken as centred (X^T X * alpha), with or without the flag."""
    rng = np.random.default_rng(3)
    for rows, cols in [(999, 70), (64, 64), (3000, 17)]:
        m = rng.normal(0.0, 1.0, (rows, cols)).astype(NP[dt])
        _check(dt, layout, rows, cols, True, m, center=False, with_mu=False)
        _check(dt, layout, rows, cols, True, m, center=True, with_mu=False)


def test_off_aligned_pointers():
    """Inputs that start one element off a 16-byte boundary (vector loads at any element
    alignment)."""
    import torch
    from raft_amd import device as dev
    rng = np.random.default_rng(5)
    for layout in (api.ROW_MAJOR, api.COL_MAJOR):
        for rows, cols in [(1000, 64), (777, 36), (500, 128)]:
            m = rng.normal(1.0, 2.0, (rows, cols)).astype(np.float32)
            stored = np.ascontiguousarray(m if layout == api.ROW_MAJOR else m.T).reshape(-1)
            mu = m.astype(np.float64).mean(axis=0).astype(np.float32)
            exp, _ = _oracle(api.F32, layout, rows, cols, True, stored, mu)
            buf = torch.zeros(rows * cols + 1, dtype=torch.float32, device="cuda")
            buf[1:] = torch.from_numpy(stored).cuda()
            out = torch.zeros(cols * cols, dtype=torch.float32, device="cuda")
            dev.cov(api.F32, layout, rows, cols, True, buf[1:], torch.from_numpy(mu).cuda(), out)
            torch.cuda.synchronize()
            assert _close(out.cpu().numpy().reshape(cols, cols), exp).all(), (layout, rows, cols)


def test_bitwise_repeatable():
    import torch
    from raft_amd import device as dev
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    for layout, rows, cols in [(api.ROW_MAJOR, 200000, 64), (api.COL_MAJOR, 100000, 128),
                               (api.ROW_MAJOR, 50000, 200)]:
        x = torch.randn(rows * cols, generator=g, device="cuda")
        mu = torch.zeros(cols, device="cuda")
        outs = []
        for _ in range(3):
            o = torch.empty(cols * cols, device="cuda")
            dev.cov(api.F32, layout, rows, cols, True, x, mu, o)
            outs.append(o)
        torch.cuda.synchronize()
        assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


def test_empty_and_errors():
    import torch
    lib = api.load()
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    out = torch.full((16,), 5.0, device="cuda")
    x = torch.ones(16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    # no columns: nothing to do; no rows: zeros, like a GEMM with k = 0
    assert lib.rmi_cov(api.F32, api.ROW_MAJOR, 4, 0, 1, 0, None, None, None, None, 0, st) == api.OK
    assert lib.rmi_cov(api.F32, api.ROW_MAJOR, 0, 4, 1, 0, None, None, out.data_ptr(),
                       ws.data_ptr(), ws.numel(), st) == api.OK
    torch.cuda.synchronize()
    assert torch.equal(out, torch.zeros_like(out))
    assert lib.rmi_cov(api.I32, api.ROW_MAJOR, 4, 4, 1, 0, x.data_ptr(), None, out.data_ptr(),
                       ws.data_ptr(), ws.numel(), st) == api.ERR_UNSUPPORTED
    assert lib.rmi_cov(99, api.ROW_MAJOR, 4, 4, 1, 0, x.data_ptr(), None, out.data_ptr(),
                       ws.data_ptr(), ws.numel(), st) == api.ERR_BAD_ENUM
    assert lib.rmi_cov(api.F32, 7, 4, 4, 1, 0, x.data_ptr(), None, out.data_ptr(),
                       ws.data_ptr(), ws.numel(), st) == api.ERR_BAD_ENUM
    assert lib.rmi_cov(api.F32, api.ROW_MAJOR, 4, 4, 1, 8, x.data_ptr(), None, out.data_ptr(),
                       ws.data_ptr(), ws.numel(), st) == api.ERR_BAD_ENUM
    assert lib.rmi_cov(api.F32, api.ROW_MAJOR, -1, 4, 1, 0, x.data_ptr(), None, out.data_ptr(),
                       ws.data_ptr(), ws.numel(), st) == api.ERR_BAD_SHAPE
    assert lib.rmi_cov(api.F32, api.ROW_MAJOR, 4, 4, 1, 0, None, None, out.data_ptr(),
                       ws.data_ptr(), ws.numel(), st) == api.ERR_NULL
    assert lib.rmi_cov(api.F32, api.ROW_MAJOR, 4, 4, 1, 0, x.data_ptr(), None, None,
                       ws.data_ptr(), ws.numel(), st) == api.ERR_NULL
    need = lib.rmi_cov_workspace_bytes(api.F32, api.ROW_MAJOR, 4, 4)
    assert need > 0
    assert lib.rmi_cov(api.F32, api.ROW_MAJOR, 4, 4, 1, 0, x.data_ptr(), None, out.data_ptr(),
                       ws.data_ptr(), need - 1, st) == api.ERR_WORKSPACE
    assert lib.rmi_cov(api.F32, api.ROW_MAJOR, 4, 4, 1, 0, x.data_ptr(), None, out.data_ptr(),
                       None, 0, st) == api.ERR_WORKSPACE
    assert lib.rmi_cov(api.F32, api.ROW_MAJOR, 4, 4, 1, 0, x.data_ptr() + 2, None, out.data_ptr(),
                       ws.data_ptr(), ws.numel(), st) == api.ERR_ALIGNMENT


def test_full_size_10m_by_64():
    """The column-statistics benchmark matrix (10,000,000 x 64 fp32, N(3, 2)): the covariance against an
    independent fp64 contraction on the device, the first 100,000 rows against the oracle as a
    problem of their own, and the centred data against x - mu."""
    import torch
    from raft_amd import device as dev
    rows, cols = 10_000_000, 64
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    x = torch.randn(rows * cols, generator=g, device="cuda").mul_(2.0).add_(3.0)
    m = x.view(rows, cols)
    mu = m.mean(dim=0, dtype=torch.float64).to(torch.float32)
    out = torch.empty(cols * cols, device="cuda")
    dev.cov(api.F32, api.ROW_MAJOR, rows, cols, True, x, mu, out)
    torch.cuda.synchronize()
    ref = torch.zeros(cols, cols, dtype=torch.float64, device="cuda")
    for c in m.split(1 << 20):
        d = (c - mu[None, :]).to(torch.float64)  # centred in fp32 first, as the library does
        ref += d.T @ d
    ref /= rows - 1
    got = out.view(cols, cols).cpu().numpy()
    assert _close(got, ref.cpu().numpy()).all()
    assert np.all(np.abs(np.diag(got) - 4.0) <= 0.06 * 4.0)
    # a slice as its own problem against the CPU oracle
    ns = 100_000
    sub = m[:ns].clone().view(-1)  # centred in place below
    sub_h = sub.cpu().numpy()
    mus = m[:ns].mean(dim=0, dtype=torch.float64).to(torch.float32)
    o2 = torch.empty(cols * cols, device="cuda")
    dev.cov(api.F32, api.ROW_MAJOR, ns, cols, False, sub, mus, o2, center=True)
    torch.cuda.synchronize()
    exp, exp_cen = _oracle(api.F32, api.ROW_MAJOR, ns, cols, False, sub_h, mus.cpu().numpy())
    assert _close(o2.view(cols, cols).cpu().numpy(), exp).all()
    assert np.array_equal(sub.cpu().numpy(), exp_cen)
