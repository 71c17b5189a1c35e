"""One-pass mean and variance (rmi_meanvar) on the GPU against the fp64 oracle: the
parameter grid of the reference's test (cpp/tests/stats/meanvar.cu:89-124) with its
statistical tolerances, both layouts, ragged shapes, shifted data, empty inputs."""
import numpy as np
import pytest

from raft_amd import _capi as api
from tests import _util as u

pytestmark = pytest.mark.gpu

NP = {api.F32: np.float32, api.F64: np.float64}


def _oracle(dt, layout, rows, cols, sample, stored):
    mean = np.zeros(cols)
    var = np.zeros(cols)
    rc = u.load_oracle().orc_meanvar(dt, layout, rows, cols, int(sample), stored.ctypes.data,
                                     mean.ctypes.data, var.ctypes.data)
    assert rc == 0
    return mean, var


def _gpu(dt, layout, rows, cols, sample, stored):
    import torch
    from raft_amd import device as dev
    x = torch.from_numpy(stored.reshape(-1)).cuda()
    tdt = torch.float32 if dt == api.F32 else torch.float64
    mean = torch.full((max(cols, 1),), 77.0, dtype=tdt, device="cuda")
    var = torch.full((max(cols, 1),), 77.0, dtype=tdt, device="cuda")
    dev.meanvar(dt, layout, rows, cols, sample, x, mean, var)
    torch.cuda.synchronize()
    return mean.cpu().numpy()[:cols], var.cpu().numpy()[:cols]


def _make(rng, dt, layout, rows, cols, mu, sd):
    m = rng.normal(mu, sd, (rows, cols)).astype(NP[dt])
    return np.ascontiguousarray(m if layout == api.ROW_MAJOR else m.T)


def _check(dt, layout, rows, cols, sample, stored, tol=1e-5):
    got_m, got_v = _gpu(dt, layout, rows, cols, sample, stored)
    exp_m, exp_v = _oracle(dt, layout, rows, cols, sample, stored)
    assert u.fp_close(got_m, exp_m, tol).all(), u.worst_rel(got_m, exp_m)
    assert u.fp_close(got_v, exp_v, tol).all(), u.worst_rel(got_v, exp_v)
    return got_m, got_v


# (mean, stddev, rows, cols, sample, row_major): cpp/tests/stats/meanvar.cu:89-124; the
# 500000 x 811 case has a test of its own below
MV = u.golden()["meanvar_tolerances"]
REF_F = [tuple(c) for c in MV["float"] if c[2] * c[3] < 10**7]
REF_D = [tuple(c) for c in MV["double"]]


@pytest.mark.parametrize("dt,case", [(api.F32, c) for c in REF_F] + [(api.F64, c) for c in REF_D])
def test_reference_grid(gpu, dt, case):
    mu, sd, rows, cols, sample, row_major = case
    layout = api.ROW_MAJOR if row_major else api.COL_MAJOR
    stored = _make(np.random.default_rng(1234), dt, layout, rows, cols, mu, sd)
    got_m, got_v = _check(dt, layout, rows, cols, sample, stored)
    # the reference's own acceptance bounds on normal data
    ns = MV["n_sigmas"]
    assert np.all(np.abs(got_m - mu) <= ns * sd / np.sqrt(rows))
    assert np.all(np.abs(got_v - sd * sd) <= ns * sd * sd * np.sqrt(2.0 / max(1, rows - 1)))


@pytest.mark.parametrize("dt", [api.F32, api.F64])
@pytest.mark.parametrize("layout", [api.ROW_MAJOR, api.COL_MAJOR])
@pytest.mark.parametrize("rows,cols", [(1, 1), (1, 7), (2, 3), (3, 1), (5, 2), (17, 5), (64, 3),
                                       (100, 33), (1000, 1), (4097, 19), (333, 1023),
                                       (20000, 6), (7, 4099), (300000, 4), (3, 100000),
                                       (150001, 37)])
def test_ragged_shapes(gpu, dt, layout, rows, cols):
    stored = _make(np.random.default_rng(rows * 31 + cols), dt, layout, rows, cols, 3.0, 2.0)
    for sample in (False, True):
        _check(dt, layout, rows, cols, sample, stored)


@pytest.mark.parametrize("layout", [api.ROW_MAJOR, api.COL_MAJOR])
def test_shifted_data(gpu, layout):
    """A mean far above the spread: sums of raw squares would cancel, the shifted sums
    and the pairwise merge do not."""
    rows, cols = 50000, 24
    stored = _make(np.random.default_rng(7), api.F64, layout, rows, cols, 1e6, 1e-2)
    _check(api.F64, layout, rows, cols, True, stored, tol=1e-7)
    stored = _make(np.random.default_rng(8), api.F32, layout, rows, cols, 1e3, 1.0)
    _check(api.F32, layout, rows, cols, True, stored)


@pytest.mark.parametrize("layout", [api.ROW_MAJOR, api.COL_MAJOR])
@pytest.mark.parametrize("rows,cols", [(671, 3000), (6710, 700), (60000, 40), (200000, 12)])
def test_outlier_first_sample(gpu, layout, rows, cols):
    """The worst case for sums that are shifted by a member of the set: every column's first
    sample lies a million standard deviations off.  Sets of up to 65536 values merge by moving
    their sums to one shift, which may cost log2(w) of the 53 bits; larger ones merge
    pairwise."""
    m = np.random.default_rng(rows + cols).normal(0.0, 1.0, (rows, cols))
    m[0, :] = 1e6
    for dt, tol in ((api.F64, 1e-8), (api.F32, 1e-5)):
        stored = np.ascontiguousarray((m if layout == api.ROW_MAJOR else m.T).astype(NP[dt]))
        _check(dt, layout, rows, cols, True, stored, tol=tol)


def test_constant_columns(gpu):
    rows, cols = 10000, 40
    stored = np.full((rows, cols), 3.25, dtype=np.float32)
    got_m, got_v = _gpu(api.F32, api.ROW_MAJOR, rows, cols, True, stored)
    assert np.all(got_m == 3.25) and np.all(got_v == 0.0)


@pytest.mark.parametrize("layout", [api.ROW_MAJOR, api.COL_MAJOR])
def test_empty(gpu, layout):
    # no columns: nothing is written; no rows: zeros
    got_m, got_v = _gpu(api.F32, layout, 5, 0, False, np.zeros(1, dtype=np.float32))
    assert got_m.size == 0 and got_v.size == 0
    got_m, got_v = _gpu(api.F32, layout, 0, 6, True, np.zeros(1, dtype=np.float32))
    assert np.all(got_m == 0) and np.all(got_v == 0)


def test_reference_large_case(gpu):
    """{10, 2, 500000 x 811, population variance, row-major}
    (cpp/tests/stats/meanvar.cu:109), checked against the oracle on a column sample and by
    the reference's statistical bound on every column."""
    import torch
    from raft_amd import device as dev
    rows, cols, mu, sd = 500000, 811, 10.0, 2.0
    g = torch.Generator(device="cuda").manual_seed(1234)
    x = torch.empty((rows, cols), dtype=torch.float32, device="cuda").normal_(mu, sd, generator=g)
    mean = torch.empty(cols, dtype=torch.float32, device="cuda")
    var = torch.empty(cols, dtype=torch.float32, device="cuda")
    dev.meanvar(api.F32, api.ROW_MAJOR, rows, cols, False, x, mean, var)
    torch.cuda.synchronize()
    got_m, got_v = mean.cpu().numpy(), var.cpu().numpy()
    assert np.all(np.abs(got_m - mu) <= 6 * sd / np.sqrt(rows))
    assert np.all(np.abs(got_v - sd * sd) <= 6 * sd * sd * np.sqrt(2.0 / (rows - 1)))
    pick = [0, 1, 405, 809, 810]
    sub = np.ascontiguousarray(x[:, pick].cpu().numpy())
    exp_m, exp_v = _oracle(api.F32, api.ROW_MAJOR, rows, len(pick), False, sub)
    assert u.fp_close(got_m[pick], exp_m).all() and u.fp_close(got_v[pick], exp_v).all()


def test_validation(gpu):
    lib = api.load()
    assert lib.rmi_meanvar(api.I32, api.ROW_MAJOR, 4, 4, 0, None, None, None, None, 0, None) \
        == api.ERR_UNSUPPORTED
    assert lib.rmi_meanvar(api.F32, 9, 4, 4, 0, None, None, None, None, 0, None) == api.ERR_BAD_ENUM
    assert lib.rmi_meanvar(api.F32, api.ROW_MAJOR, -1, 4, 0, None, None, None, None, 0, None) \
        == api.ERR_BAD_SHAPE
    assert lib.rmi_meanvar(api.F32, api.ROW_MAJOR, 4, 4, 0, None, None, None, None, 0, None) \
        == api.ERR_NULL


# 16-bit data (f16, bf16): the arithmetic is f64, mean and variance are rounded once to the
# data's type; the oracle reads the same stored bits.
@pytest.mark.parametrize("dt", [api.F16, api.BF16])
@pytest.mark.parametrize("layout", [api.ROW_MAJOR, api.COL_MAJOR])
@pytest.mark.parametrize("rows,cols", [(1, 5), (17, 3), (1000, 64), (4097, 19), (333, 1023),
                                       (200000, 8), (9, 4100)])
def test_half_types(gpu, dt, layout, rows, cols):
    import torch
    from raft_amd import device as dev
    rng = np.random.default_rng(rows + cols)
    f = rng.normal(1.5, 2.0, (rows, cols)).astype(np.float32)
    f = np.ascontiguousarray(f if layout == api.ROW_MAJOR else f.T)
    stored = f.astype(np.float16).view(np.uint16) if dt == api.F16 else u.to_bf16(f.reshape(-1))
    stored = np.ascontiguousarray(stored.reshape(-1))
    x = torch.from_numpy(stored.view(np.int16)).cuda()
    mean = torch.zeros(cols, dtype=torch.int16, device="cuda")
    var = torch.zeros(cols, dtype=torch.int16, device="cuda")
    for sample in (False, True):
        dev.meanvar(dt, layout, rows, cols, sample, x, mean, var)
        torch.cuda.synchronize()
        raw_m = mean.cpu().numpy().view(np.uint16)
        raw_v = var.cpu().numpy().view(np.uint16)
        if dt == api.F16:
            got_m, got_v = raw_m.view(np.float16).astype(np.float64), raw_v.view(np.float16).astype(np.float64)
        else:
            got_m, got_v = u.from_bf16(raw_m).astype(np.float64), u.from_bf16(raw_v).astype(np.float64)
        exp_m, exp_v = _oracle(dt, layout, rows, cols, sample, stored)
        # rounded once from f64: the correctly rounded oracle value or the number next to it
        assert u.ulp16_ok(dt, raw_m, exp_m).all(), u.worst_rel(got_m, exp_m)
        assert u.ulp16_ok(dt, raw_v, exp_v).all(), u.worst_rel(got_v, exp_v)
