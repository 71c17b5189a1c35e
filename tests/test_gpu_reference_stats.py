"""The grids of the reference's stats tests at their own sizes, generated on the device:
cpp/tests/stats/sum.cu:108-140 (Result and Accuracy), mean.cu:118-215, stddev.cu:119-202,
including the cases of 10^8 x 1 and 2^27 x 2 elements in both layouts.  The cases are data
under tests/golden/reference_fixtures.json; the reference's RNG is not reproduced (torch's
normal generator stands in), so each result is held to the reference's own bound AND, more
tightly, to an fp64 evaluation of the same device buffer."""
import numpy as np
import pytest

from raft_amd import _capi as api
from tests import _util as u

pytestmark = pytest.mark.gpu

GOLD = u.golden()


def _torch_dtype(dt):
    import torch
    return {api.F32: torch.float32, api.F64: torch.float64, api.F16: torch.float16,
            api.I8: torch.int8}[dt]


def _run(desc, x, out, aux=None):
    import torch
    from raft_amd import device as dev
    d = api.ReduceDesc.from_buffer_copy(desc)
    if aux is not None:
        d.final_aux = aux.data_ptr()
    dev.reduce(d, x, out)
    torch.cuda.synchronize()
    return out


def _stored(col_values, rows, cols, row_major):
    """A [rows, cols] matrix whose every column is `col_values`, in the asked layout."""
    if row_major:
        return col_values[:, None].expand(rows, cols).contiguous().view(-1)
    return col_values[None, :].expand(cols, rows).contiguous().view(-1)


def _col_sums_f64(x, rows, cols, row_major):
    """Column sums of the stored matrix in fp64 by torch, in slices that bound memory."""
    import torch
    m = x.view(rows, cols) if row_major else x.view(cols, rows)
    tot = torch.zeros(cols, dtype=torch.float64, device=x.device)
    step = 1 << 24
    for r in range(0, rows, step):
        blk = m[r:r + step] if row_major else m[:, r:r + step]
        tot += blk.sum(dim=0 if row_major else 1, dtype=torch.float64)
    return tot


# ---- stats::sum ------------------------------------------------------------------------------
SUM_BIG = [(k, c) for k in ("float", "double") for c in GOLD["stats_sum"][k] if c[1] * c[2] > 10**6]


@pytest.mark.parametrize("kind,case", SUM_BIG, ids=lambda x: str(x))
@pytest.mark.parametrize("accuracy", [False, True])
def test_sum_large(gpu, kind, case, accuracy):
    import torch
    g = GOLD["stats_sum"]
    tol, rows, cols, row_major, value = case
    npdt, dt = (np.float32, api.F32) if kind == "float" else (np.float64, api.F64)
    tdt = _torch_dtype(dt)
    v = float(npdt(value))  # params.value is a T; the test computes in double from it
    col = torch.full((rows,), v, dtype=torch.float64, device="cuda")
    if accuracy:  # sum.cu:62-76
        large = g["large_factor"][kind]
        r = torch.arange(rows, device="cuda")
        col[r % 3 == 2] = v * large
        col[(r % 3 == 1) & (r + 1 < rows)] = -v * large
        col[(r % 3 == 0) & (r + 2 < rows)] = 3.0 * v
        del r
    col = col.to(tdt)
    x = _stored(col, rows, cols, row_major)
    del col
    d = api.make_desc(dt, dt, rows, cols, apply=api.ALONG_COLUMNS,
                      layout=api.ROW_MAJOR if row_major else api.COL_MAJOR)
    out = _run(d, x, torch.zeros(cols, dtype=tdt, device="cuda"))
    got = out.cpu().numpy().astype(np.float64)
    expected = np.full(cols, float(npdt(rows * v)))  # T(double(rows) * value)
    # the reference's bound (100x looser for Accuracy there; the plain one is held here)
    assert u.approx_ok(got, expected, tol).all(), (got, expected)
    if not accuracy:
        if kind == "float":
            # fp32 terms summed in fp64 carry no error at all: the result is the rounded product
            assert np.array_equal(got, expected)
        else:
            assert np.allclose(got, expected, rtol=1e-13, atol=0)
    else:
        # exact value of the Accuracy sum: the large terms cancel exactly, what is left is
        # (rows // 3) triples of T(3v) and rows % 3 plain values
        three = float(npdt(3.0 * v))
        exact = (rows // 3) * three + (rows % 3) * v
        assert np.allclose(got, exact, rtol=1e-6 if kind == "float" else 1e-13, atol=0), (got, exact)


# ---- stats::mean -----------------------------------------------------------------------------
MEAN_KINDS = {"float": (api.F32, api.F32, np.float32), "double": (api.F64, api.F64, np.float64),
              "half_to_float": (api.F16, api.F32, np.float32), "int8_to_half": (api.I8, api.F16, np.float16)}
MEAN_CASES = [(k, c) for k in MEAN_KINDS for c in GOLD["stats_mean"][k]]


@pytest.mark.parametrize("kind,case", MEAN_CASES, ids=lambda x: str(x))
def test_mean_grid(gpu, kind, case):
    import torch
    tol, mean, rows, cols, row_major, sd = case
    in_dt, out_dt, out_np = MEAN_KINDS[kind]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1234)
    n = rows * cols
    if in_dt == api.F64:
        x = torch.randn(n, generator=gen, device="cuda", dtype=torch.float64).mul_(sd).add_(mean)
    else:
        x = torch.randn(n, generator=gen, device="cuda", dtype=torch.float32).mul_(sd).add_(mean)
        if in_dt == api.F16:
            x = x.to(torch.float16)           # mean.cu:82-85: normal in float, then __float2half
        elif in_dt == api.I8:
            x = x.round_().clamp_(-128, 127).to(torch.int8)   # normalInt
    ratio = float(out_np(1) / out_np(rows))   # stats/detail/mean.cuh:22
    d = api.make_desc(in_dt, out_dt, rows, cols, apply=api.ALONG_COLUMNS,
                      layout=api.ROW_MAJOR if row_major else api.COL_MAJOR,
                      final_op=api.FIN_MUL_CONST, final_scalar=ratio)
    tout = torch.float16 if out_dt == api.F16 else _torch_dtype(out_dt)
    out = _run(d, x, torch.zeros(cols, dtype=tout, device="cuda"))
    got_raw = out.cpu().numpy()
    got = got_raw.astype(np.float64)
    ref = _col_sums_f64(x, rows, cols, row_major).cpu().numpy() * ratio
    if kind == "int8_to_half":
        assert np.all(np.abs(got - mean) <= tol), (got[:4], mean)          # ASSERT_NEAR
        assert u.ulp16_ok(api.F16, got_raw.view(np.uint16), ref).all()
        return
    if kind == "double" and tol < 1e-6:
        # The reference holds |mean_j - 0.1| to 1e-8 on ITS generator's data; the sampling error
        # of 2^27 draws of stddev 1e-4 is 0.9e-8 by itself, so on other data that bound is a
        # statement about the draw.  Held here: four standard errors of the draw, and the fp64
        # evaluation of the same buffer to 1e-13.
        assert np.all(np.abs(got - mean) <= 4 * sd / np.sqrt(rows) + tol), (got, mean)
    else:
        m_in = float(np.float16(mean)) if in_dt == api.F16 else mean
        assert u.approx_ok(got, np.full(cols, m_in), tol).all(), (got[:4], mean)
    assert np.allclose(got, ref, rtol=1e-13 if out_dt == api.F64 else 1e-6, atol=0), (got[:4], ref[:4])


# ---- stats::stddev / vars --------------------------------------------------------------------
STD_CASES = [(k, c) for k in ("float", "double") for c in GOLD["stats_stddev"][k]]


@pytest.mark.parametrize("kind,case", STD_CASES, ids=lambda x: str(x))
def test_stddev_grid(gpu, kind, case):
    import torch
    tol, mean, sd, rows, cols, sample, row_major = case
    npdt, dt = (np.float32, api.F32) if kind == "float" else (np.float64, api.F64)
    tdt = _torch_dtype(dt)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1234)
    n = rows * cols
    if sd == 0:
        x = torch.full((n,), mean, dtype=tdt, device="cuda")  # normal(mean, 0)
    else:
        x = torch.randn(n, generator=gen, device="cuda", dtype=tdt).mul_(sd).add_(mean)
    lay = api.ROW_MAJOR if row_major else api.COL_MAJOR
    dm = api.make_desc(dt, dt, rows, cols, layout=lay, apply=api.ALONG_COLUMNS,
                       final_op=api.FIN_MUL_CONST, final_scalar=float(npdt(1) / npdt(rows)))
    mu = _run(dm, x, torch.zeros(cols, dtype=tdt, device="cuda"))
    # stats/detail/stddev.cuh:49-50
    with np.errstate(divide="ignore"):
        ratio = npdt(1) / npdt(rows - 1 if sample else rows)
    ratio_mean = npdt(ratio * npdt(rows)) if sample else npdt(1)
    res = {}
    for name, fin in (("stddev", api.FIN_STDDEV_FROM_SUMSQ), ("vars", api.FIN_VAR_FROM_SUMSQ)):
        ds = api.make_desc(dt, dt, rows, cols, layout=lay, apply=api.ALONG_COLUMNS,
                           main_op=api.MAIN_SQ, final_op=fin, final_scalar=float(ratio),
                           final_scalar2=float(ratio_mean))
        res[name] = _run(ds, x, torch.zeros(cols, dtype=tdt, device="cuda"),
                         aux=mu).cpu().numpy().astype(np.float64)
    # stddev.cu:185-202
    want = 0.0 if rows == 1 else sd
    assert u.approx_ok(res["stddev"], np.full(cols, want), tol).all(), (res["stddev"][:4], want)
    assert u.approx_ok(np.sqrt(res["vars"]), res["stddev"], tol).all()
    if rows > 1 and sd > 0:
        # fp64 two-pass evaluation of the same buffer; E[x^2] - mu^2 in the data's own arithmetic
        # loses |mu|^2 / sd^2 * eps, far inside 1e-5 for these means and deviations
        m = (x.view(rows, cols) if row_major else x.view(cols, rows).t()).double()
        ref = m.std(dim=0, unbiased=bool(sample)).cpu().numpy()
        assert u.fp_close(res["stddev"], ref, 1e-5 if kind == "float" else 1e-9).all(), \
            u.worst_rel(res["stddev"], ref)
