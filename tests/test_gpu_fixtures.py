"""The reference's own known-answer fixtures for the reduction path, run through the
C ABI on the GPU.  Each test names the reference test file and lines it restates."""
import numpy as np
import pytest

from raft_amd import _capi as api
from tests import _util as u

pytestmark = pytest.mark.gpu

GOLD = u.golden()


# cpp/tests/linalg/reduce.cu:108-177 (simpleTest): data 1..12 as 3x4, max_op, init 0.
@pytest.mark.parametrize("case", list(GOLD["reduce_simple_max"]["expected"]))
@pytest.mark.parametrize("dt,npdt", [(api.F32, np.float32), (api.F64, np.float64)])
def test_reduce_simple_max(gpu, case, dt, npdt):
    g = GOLD["reduce_simple_max"]
    layout, apply = u.LAYOUT_AXIS[case]
    expected = g["expected"][case]
    data = np.array(g["data"], dtype=npdt)
    d = api.make_desc(dt, dt, g["rows"], g["cols"], layout=layout, apply=apply,
                      reduce_op=api.RED_MAX)
    got = u.gpu_reduce(d, data)
    assert got.tolist() == [float(e) for e in expected]


# cpp/tests/matrix/argmax.cu:71-75 and argmin.cu:71-75: 3x4 literal, key-only output.
ARG = GOLD["matrix_arg"]
ARG_DATA = ARG["data"]


@pytest.mark.parametrize("dt,npdt", [(api.F32, np.float32), (api.F64, np.float64)])
def test_matrix_argmax_argmin_fixture(gpu, dt, npdt):
    data = np.array(ARG_DATA, dtype=npdt)
    dmax = api.make_desc(dt, api.I32, 3, 4, main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX,
                         final_op=api.FIN_KEY, init_i=0, init_f=-np.inf)
    assert u.gpu_reduce(dmax, data).tolist() == ARG["argmax"]
    dmin = api.make_desc(dt, api.I32, 3, 4, main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMIN,
                         final_op=api.FIN_KEY, init_i=0, init_f=np.inf)
    assert u.gpu_reduce(dmin, data).tolist() == ARG["argmin"]


# cpp/tests/util/reduction.cu:167-171,179-181: the literal 64-vector.
W64 = GOLD["wave_vector64"]
VEC64 = W64["data"]


def test_wave_reduction_vector(gpu):
    x = np.array(VEC64, dtype=np.int32)
    for red, init, want in [(api.RED_MIN, 2**62, W64["min"]), (api.RED_MAX, -2**62, W64["max"]),
                            (api.RED_ADD, 0, W64["sum"])]:
        d = api.make_desc(api.I32, api.I64, 1, 64, reduce_op=red, init_i=init)
        assert u.gpu_reduce(d, x).tolist() == [want]
    xf = x.astype(np.float32)
    d = api.make_desc(api.F32, api.KVP_I32_F32, 1, 64, main_op=api.MAIN_KVP,
                      reduce_op=api.RED_ARGMAX, init_i=0, init_f=-np.inf)
    r = u.gpu_reduce(d, xf)
    assert [int(r["key"][0]), float(r["value"][0])] == W64["argmax"]
    d = api.make_desc(api.F32, api.KVP_I32_F32, 1, 64, main_op=api.MAIN_KVP,
                      reduce_op=api.RED_ARGMIN, init_i=0, init_f=np.inf)
    r = u.gpu_reduce(d, xf)
    assert [int(r["key"][0]), float(r["value"][0])] == W64["argmin"]


# cpp/tests/stats/sum.cu:50-98,108-140: the reference's grid, plain ("Result") and with the
# (3v, -vL, +vL) triples ("Accuracy"); the column sums must be rows * value.  The cases of 10^8
# and 2^27 rows are generated on the device in tests/test_gpu_reference_stats.py.
from tests.test_oracle import SUM_SMALL, sum_case_matrix  # noqa: E402


@pytest.mark.parametrize("kind,case", SUM_SMALL, ids=lambda x: str(x))
@pytest.mark.parametrize("accuracy", [False, True])
def test_sum_grid(gpu, kind, case, accuracy):
    g = GOLD["stats_sum"]
    tol, rows, cols, row_major, value = case
    npdt, dt = (np.float32, api.F32) if kind == "float" else (np.float64, api.F64)
    m = sum_case_matrix(npdt, rows, cols, value, g["large_factor"][kind] if accuracy else None)
    flat = np.ascontiguousarray(m.reshape(-1) if row_major else m.T.reshape(-1))
    d = api.make_desc(dt, dt, rows, cols, apply=api.ALONG_COLUMNS,
                      layout=api.ROW_MAJOR if row_major else api.COL_MAJOR)
    got = u.gpu_reduce(d, flat).astype(np.float64)
    expected = np.full(cols, float(npdt(rows * float(npdt(value)))))
    # the reference allows 100 * tolerance for the Accuracy variant; this build holds the
    # plain tolerance for both
    assert u.approx_ok(got, expected, tol).all(), (got[:4], expected[:4])


# Constant data => stddev 0, one row => 0, sqrt(vars) == stddev (what
# cpp/tests/stats/stddev.cu:148-149,187-202 checks; its own 2^27-row cases run at full size in
# tests/test_gpu_reference_stats.py).
@pytest.mark.parametrize("rows,cols", [(1, 1), (1, 257), (31, 1), (4096, 64)])
@pytest.mark.parametrize("sample", [False, True])
def test_stddev_constant_data(gpu, rows, cols, sample):
    v = np.float32(1.25)
    data = np.full(rows * cols, v, dtype=np.float32)
    ratio = np.float32(1.0) / np.float32(rows)
    dm = api.make_desc(api.F32, api.F32, rows, cols, apply=api.ALONG_COLUMNS,
                       final_op=api.FIN_MUL_CONST, final_scalar=float(ratio))
    mu = u.gpu_reduce(dm, data)
    assert np.allclose(mu, v, rtol=1e-6)
    if sample and rows == 1:
        return  # 1/(N-1) is infinite; the reference does not run this case either
    r = np.float32(1.0) / np.float32(rows - 1 if sample else rows)
    rm = np.float32(r * np.float32(rows)) if sample else np.float32(1.0)
    ds = api.make_desc(api.F32, api.F32, rows, cols, apply=api.ALONG_COLUMNS,
                       main_op=api.MAIN_SQ, final_op=api.FIN_STDDEV_FROM_SUMSQ,
                       final_scalar=float(r), final_scalar2=float(rm))
    sd = u.gpu_reduce(ds, data, aux_raw=mu)
    assert np.all(np.abs(sd) <= 2e-3), sd[:4]
    dv = api.make_desc(api.F32, api.F32, rows, cols, apply=api.ALONG_COLUMNS,
                       main_op=api.MAIN_SQ, final_op=api.FIN_VAR_FROM_SUMSQ,
                       final_scalar=float(r), final_scalar2=float(rm))
    var = u.gpu_reduce(dv, data, aux_raw=mu)
    # cpp/tests/stats/stddev.cu:198-202: sqrt(vars) == stddev
    assert np.allclose(np.sqrt(var), sd, atol=1e-6)


# cpp/tests/linalg/map_then_reduce.cu:140-169: U[2,3) of length 1237 with 1 planted at
# [42] and 5 at [337]; min -> 1, max -> 5 exactly.  :101-125: sum within 1e-3.
def test_map_reduce_planted(gpu):
    import torch
    from raft_amd import device as dev
    rng = np.random.default_rng(1234)
    x = rng.uniform(2.0, 3.0, 1237).astype(np.float32)
    x[42], x[337] = 1.0, 5.0
    xt = torch.from_numpy(x).cuda()
    out = torch.zeros(1, dtype=torch.float32, device="cuda")
    d = api.make_desc(api.F32, api.F32, 0, 0, reduce_op=api.RED_MIN, init_f=np.inf)
    dev.map_reduce(d, x.size, xt, out)
    assert out.item() == 1.0
    d = api.make_desc(api.F32, api.F32, 0, 0, reduce_op=api.RED_MAX, init_f=-np.inf)
    dev.map_reduce(d, x.size, xt, out)
    assert out.item() == 5.0
    big = rng.uniform(-1.0, 1.0, 1 << 20).astype(np.float32)
    bt = torch.from_numpy(big).cuda()
    d = api.make_desc(api.F32, api.F32, 0, 0)
    dev.map_reduce(d, big.size, bt, out)
    assert abs(out.item() - big.astype(np.float64).sum()) <= 1e-3
