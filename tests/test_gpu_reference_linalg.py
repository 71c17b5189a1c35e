"""The grids of the reference's linalg tests for this path, case by case as data from
tests/golden/reference_fixtures.json: cpp/tests/linalg/coalesced_reduction.cu:109-139,
strided_reduction.cu:93-102, norm.cu:234-292, map_then_reduce.cu:100-125.  Each case runs
the call sequence of the reference's test (inplace = false, then inplace = true on the same
output where it does that) and is held to the reference's own comparator and tolerance
against the fp64 oracle; the reference's RNG is not reproduced (numpy's uniform stands in)."""
import itertools

import numpy as np
import pytest

from raft_amd import _capi as api
from tests import _util as u

pytestmark = pytest.mark.gpu

GOLD = u.golden()
KINDS = {"float": (api.F32, np.float32), "double": (api.F64, np.float64)}


def _twice(desc, data, tol, label):
    """inplace = false, then inplace = true on the same output (coalesced_reduction.cu:69-93)."""
    first = u.gpu_reduce(desc, data)
    exp1 = u.oracle_reduce(desc, data)
    assert u.approx_ok(u.decode_out(desc.out_dtype, first), exp1, tol).all(), label
    d2 = api.ReduceDesc.from_buffer_copy(desc)
    d2.inplace = 1
    second = u.gpu_reduce(d2, data, old_raw=first)
    exp2 = u.oracle_reduce(d2, data, old=u.decode_out(desc.out_dtype, first))
    assert u.approx_ok(u.decode_out(desc.out_dtype, second), exp2, tol).all(), label + " inplace"


COAL = [(k, c) for k in KINDS for c in GOLD["linalg_coalesced_reduction"][k]]


@pytest.mark.parametrize("kind,case", COAL, ids=lambda x: str(x))
def test_coalesced_reduction_grid(gpu, kind, case):
    tol, rows, cols = case
    dt, npdt = KINDS[kind]
    data = np.random.default_rng(1234).uniform(-1, 1, rows * cols).astype(npdt)
    d = api.make_desc(dt, dt, rows, cols, apply=api.ALONG_ROWS, main_op=api.MAIN_SQ)
    _twice(d, data, tol, f"coalesced {rows}x{cols}")


STRI = [(k, c) for k in KINDS for c in GOLD["linalg_strided_reduction"][k]]


@pytest.mark.parametrize("kind,case", STRI, ids=lambda x: str(x))
def test_strided_reduction_grid(gpu, kind, case):
    tol, rows, cols = case
    dt, npdt = KINDS[kind]
    data = np.random.default_rng(1234).uniform(-1, 1, rows * cols).astype(npdt)
    d = api.make_desc(dt, dt, rows, cols, apply=api.ALONG_COLUMNS, main_op=api.MAIN_SQ)
    _twice(d, data, tol, f"strided {rows}x{cols}")


NORM = GOLD["linalg_norm"]
NORM_TYPES = {"float": (api.F32, api.F32, np.float32), "double": (api.F64, api.F64, np.float64),
              "half_to_float": (api.F16, api.F32, np.float16)}


@pytest.mark.parametrize("kind", list(NORM_TYPES))
@pytest.mark.parametrize("axis", ["row", "col"])
@pytest.mark.parametrize("norm", NORM["norms"])
@pytest.mark.parametrize("do_sqrt", NORM["do_sqrt"])
def test_norm_grid(gpu, kind, axis, norm, do_sqrt):
    in_dt, out_dt, npdt = NORM_TYPES[kind]
    tol = NORM["tolerance"][kind]
    main = api.MAIN_ABS if norm == "L1" else api.MAIN_SQ
    rng = np.random.default_rng(1234)
    for rows, cols in itertools.product(NORM[axis]["rows"], NORM[axis]["cols"]):
        data = rng.uniform(-1, 1, rows * cols).astype(npdt)
        d = api.make_desc(in_dt, out_dt, rows, cols,
                          apply=api.ALONG_ROWS if axis == "row" else api.ALONG_COLUMNS, main_op=main,
                          final_op=api.FIN_SQRT if do_sqrt else api.FIN_IDENTITY)
        got = u.decode_out(out_dt, u.gpu_reduce(d, data))
        exp = u.oracle_reduce(d, data)
        assert u.approx_ok(got, exp, tol).all(), (kind, axis, norm, do_sqrt, rows, cols, u.worst_rel(got, exp))
        # and what the mathematics fixes, independent of the oracle
        m = data.astype(np.float64).reshape(rows, cols)
        ref = np.abs(m).sum(axis=1 if axis == "row" else 0) if norm == "L1" else \
            (m * m).sum(axis=1 if axis == "row" else 0)
        assert np.allclose(got, np.sqrt(ref) if do_sqrt else ref, rtol=1e-6 if out_dt == api.F32 else 1e-12)


@pytest.mark.parametrize("in_t,out_t,tol,n", GOLD["linalg_map_then_reduce"]["cases"])
def test_map_then_sum_reduce_grid(gpu, in_t, out_t, tol, n):
    import torch
    from raft_amd import device as dev
    in_dt, npdt = KINDS[in_t]
    out_dt, _ = KINDS[out_t]
    x = np.random.default_rng(1234).uniform(-1, 1, n).astype(npdt)
    xt = torch.from_numpy(x).cuda()
    out = torch.zeros(1, dtype=torch.float32 if out_dt == api.F32 else torch.float64, device="cuda")
    d = api.make_desc(in_dt, out_dt, 0, 0)
    dev.map_reduce(d, n, xt, out)
    torch.cuda.synchronize()
    want = x.astype(np.float64).sum()
    assert u.approx_ok(np.array([out.item()]), np.array([want]), tol).all(), (out.item(), want)
    # far inside the reference's tolerance: the sum is deterministic and carried in fp64
    assert abs(out.item() - want) <= (1e-6 if out_dt == api.F32 else 1e-12) * max(1.0, abs(want)) + \
        (np.finfo(np.float32).eps * abs(want) if out_dt == api.F32 else 0.0)
