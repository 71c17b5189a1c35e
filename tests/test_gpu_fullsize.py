"""The benchmark shapes at their full sizes, checked through properties that do not
need a CPU pass over gigabytes: linearity, a checksum of checksums, agreement between
different launch plans, the first-maximum rule, and the oracle on a slice of the rows.
Inputs are generated on the device from fixed seeds."""
import ctypes as C

import numpy as np
import pytest

from raft_amd import _capi as api
from tests import _util as u

pytestmark = pytest.mark.gpu


def _gen(seed):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return g


def _run(desc, x, out, aux=None):
    import torch
    from raft_amd import device as dev
    d = api.ReduceDesc.from_buffer_copy(desc)
    if aux is not None:
        d.final_aux = aux.data_ptr()
    dev.reduce(d, x, out)
    torch.cuda.synchronize()
    return out


def _host(t):
    import torch
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


# config 1: row sums of fp32 10000 x 256, U[-1,1), seed 0 -- small enough for the oracle
def test_cfg1_row_sum_full(gpu):
    import torch
    rows, cols = 10000, 256
    x = torch.rand(rows * cols, generator=_gen(0), device="cuda") * 2 - 1
    d = api.make_desc(api.F32, api.F32, rows, cols)
    out = _run(d, x, torch.zeros(rows, device="cuda"))
    exp = u.oracle_reduce(d, _host(x))
    assert u.fp_close(_host(out), exp).all(), u.worst_rel(_host(out), exp)


# config 2: L2 row norms of fp32 1,000,000 x 128, N(0,1)
def test_cfg2_l2_row_norm_full(gpu):
    import torch
    rows, cols = 1000000, 128
    x = torch.randn(rows * cols, generator=_gen(2), device="cuda")
    d = api.make_desc(api.F32, api.F32, rows, cols, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
    out = _run(d, x, torch.zeros(rows, device="cuda"))
    # oracle on the first and last 20000 rows
    for sl in (slice(0, 20000), slice(rows - 20000, rows)):
        sub = x.view(rows, cols)[sl].contiguous()
        ds = api.make_desc(api.F32, api.F32, 20000, cols, main_op=api.MAIN_SQ,
                           final_op=api.FIN_SQRT)
        exp = u.oracle_reduce(ds, _host(sub).reshape(-1))
        assert u.fp_close(_host(out[sl]), exp).all()
    # scaling: ||a x|| = |a| ||x|| exactly for a power of two
    out2 = _run(d, x * 4.0, torch.zeros(rows, device="cuda"))
    assert torch.equal(out2, out * 4.0)
    # sum over rows of ||x_r||^2 equals the squared Frobenius norm (checksum of checksums)
    d1 = api.make_desc(api.F32, api.F64, 1, rows * cols, main_op=api.MAIN_SQ)
    tot = _run(d1, x, torch.zeros(1, dtype=torch.float64, device="cuda")).item()
    assert abs((out.double() ** 2).sum().item() - tot) <= 1e-6 * tot


# config 3: column mean then column stddev of fp32 10,000,000 x 64, N(3,2)
def test_cfg3_column_mean_stddev_full(gpu):
    import torch
    rows, cols = 10000000, 64
    x = torch.randn(rows * cols, generator=_gen(3), device="cuda").mul_(2.0).add_(3.0)
    ratio = float(np.float32(1.0) / np.float32(rows))
    dm = api.make_desc(api.F32, api.F32, rows, cols, apply=api.ALONG_COLUMNS,
                       final_op=api.FIN_MUL_CONST, final_scalar=ratio)
    mu = _run(dm, x, torch.zeros(cols, device="cuda"))
    for sample in (False, True):
        r = np.float32(1.0) / np.float32(rows - 1 if sample else rows)
        rm = np.float32(r * np.float32(rows)) if sample else np.float32(1.0)
        ds = api.make_desc(api.F32, api.F32, rows, cols, apply=api.ALONG_COLUMNS,
                           main_op=api.MAIN_SQ, final_op=api.FIN_STDDEV_FROM_SUMSQ,
                           final_scalar=float(r), final_scalar2=float(rm))
        sd = _run(ds, x, torch.zeros(cols, device="cuda"), aux=mu)
        # against an independent fp64 evaluation on the device, two-pass formula
        xv = x.view(rows, cols)
        m64 = torch.zeros(cols, dtype=torch.float64, device="cuda")
        for c in xv.split(1 << 21):
            m64 += c.sum(dim=0, dtype=torch.float64)
        m64 /= rows
        ss = torch.zeros(cols, dtype=torch.float64, device="cuda")
        for c in xv.split(1 << 21):
            ss += ((c.double() - m64) ** 2).sum(dim=0)
        ref = torch.sqrt(ss / (rows - 1 if sample else rows))
        assert u.fp_close(_host(mu), _host(m64)).all(), u.worst_rel(_host(mu), _host(m64))
        assert u.fp_close(_host(sd), _host(ref)).all(), u.worst_rel(_host(sd), _host(ref))
    # the same column sums from a different route: one-row reductions of column slices
    # are not available without a transpose, so use linearity instead:
    # sum_rows(x) == sum_rows(x[:half]) + sum_rows(x[half:]) to fp64 accuracy
    dsum = api.make_desc(api.F32, api.F64, rows, cols, apply=api.ALONG_COLUMNS)
    full = _run(dsum, x, torch.zeros(cols, dtype=torch.float64, device="cuda"))
    h = rows // 2
    dh = api.make_desc(api.F32, api.F64, h, cols, apply=api.ALONG_COLUMNS)
    a = _run(dh, x.view(rows, cols)[:h], torch.zeros(cols, dtype=torch.float64, device="cuda"))
    b = _run(dh, x.view(rows, cols)[h:], torch.zeros(cols, dtype=torch.float64, device="cuda"))
    assert torch.allclose(full, a + b, rtol=1e-12, atol=0)
    # and the oracle on the first 100000 rows as a problem of its own
    ns = 100000
    sub = x.view(rows, cols)[:ns].contiguous()
    dsub = api.make_desc(api.F32, api.F32, ns, cols, apply=api.ALONG_COLUMNS)
    got = _run(dsub, sub, torch.zeros(cols, device="cuda"))
    exp = u.oracle_reduce(dsub, _host(sub).reshape(-1))
    assert u.fp_close(_host(got), exp).all()


# config 4: row argmax of fp32 65536 x 32000, exact ties injected in 1% of the rows
def test_cfg4_row_argmax_full(gpu):
    import torch
    rows, cols = 65536, 32000
    g = _gen(4)
    x = torch.randn(rows, cols, generator=g, device="cuda")
    n_tie = rows // 100
    tie_rows = torch.randperm(rows, generator=g, device="cuda")[:n_tie]
    mx = x[tie_rows].amax(dim=1)
    for j in range(3):
        pos = torch.randint(0, cols, (n_tie,), generator=g, device="cuda")
        keep = torch.rand(n_tie, generator=g, device="cuda") < (1.0 if j == 0 else 0.5)
        x[tie_rows[keep], pos[keep]] = mx[keep]
    d = api.make_desc(api.F32, api.KVP_I32_F32, rows, cols, main_op=api.MAIN_KVP,
                      reduce_op=api.RED_ARGMAX, init_i=0, init_f=-np.inf)
    out = _run(d, x, torch.zeros(rows * 2, dtype=torch.int32, device="cuda")).view(rows, 2)
    keys = out[:, 0].to(torch.int64)
    vals = out[:, 1].contiguous().view(torch.float32)
    ar = torch.arange(cols, device="cuda", dtype=torch.int64)
    tied = 0
    for r0 in range(0, rows, 4096):
        blk = x[r0:r0 + 4096]
        m = blk.amax(dim=1)
        eq = blk == m[:, None]
        first = torch.where(eq, ar[None, :], torch.full((), cols, device="cuda",
                                                        dtype=torch.int64)).amin(dim=1)
        tied += int((eq.sum(dim=1) > 1).sum().item())
        assert torch.equal(first, keys[r0:r0 + 4096]), "lowest index of the maximum"
        assert torch.equal(m, vals[r0:r0 + 4096])
    assert tied >= n_tie // 2, "the input must really contain ties"
    # key-only route and a different launch plan give the same indices
    dk = api.make_desc(api.F32, api.I32, rows, cols, main_op=api.MAIN_KVP,
                       reduce_op=api.RED_ARGMAX, final_op=api.FIN_KEY, init_i=0, init_f=-np.inf,
                       plan_hint=api.PLAN_ROW_BLOCK)
    k2 = _run(dk, x, torch.zeros(rows, dtype=torch.int32, device="cuda"))
    assert torch.equal(k2.to(torch.int64), keys)
    # the oracle on a slice of the tied rows
    pick = tie_rows[:64].sort().values
    sub = x[pick].contiguous()
    dsub = api.make_desc(api.F32, api.KVP_I32_F32, 64, cols, main_op=api.MAIN_KVP,
                         reduce_op=api.RED_ARGMAX, init_i=0, init_f=-np.inf)
    ek, ev = u.oracle_reduce(dsub, _host(sub).reshape(-1))
    assert np.array_equal(_host(keys[pick]), ek)
    assert np.array_equal(_host(vals[pick]).astype(np.float64), ev)


# config 5: int8 4096 x 16384 and 16,777,216 x 8 into int64 (bit-exact), bf16 8 x 4,194,304
def test_cfg5_mixed_precision_full(gpu):
    import torch
    # 5a
    rows, cols = 4096, 16384
    x = torch.randint(-128, 128, (rows * cols,), generator=_gen(5), device="cuda",
                      dtype=torch.int8)
    d = api.make_desc(api.I8, api.I64, rows, cols)
    out = _run(d, x, torch.zeros(rows, dtype=torch.int64, device="cuda"))
    exp = u.oracle_reduce(d, _host(x))
    assert np.array_equal(_host(out), exp)
    # 5b: oracle on the first 2M rows, checksum of checksums on all
    rows, cols = 16777216, 8
    x = torch.randint(-128, 128, (rows * cols,), generator=_gen(6), device="cuda",
                      dtype=torch.int8)
    d = api.make_desc(api.I8, api.I64, rows, cols)
    out = _run(d, x, torch.zeros(rows, dtype=torch.int64, device="cuda"))
    ns = 1 << 21
    dsub = api.make_desc(api.I8, api.I64, ns, cols)
    exp = u.oracle_reduce(dsub, _host(x[: ns * cols]))
    assert np.array_equal(_host(out[:ns]), exp)
    d1 = api.make_desc(api.I8, api.I64, 1, rows * cols)
    tot = _run(d1, x, torch.zeros(1, dtype=torch.int64, device="cuda")).item()
    assert int(out.sum().item()) == tot
    # an odd row count exercises the tail rows that do not fill a 16-byte vector
    d_odd = api.make_desc(api.I8, api.I64, rows - 1, cols)
    out_odd = _run(d_odd, x, torch.zeros(rows - 1, dtype=torch.int64, device="cuda"))
    assert torch.equal(out_odd, out[:-1])
    # 5c: bf16 rows of 4 Mi elements, two-pass split; the oracle handles 32 Mi elements
    rows, cols = 8, 4194304
    xf = torch.rand(rows * cols, generator=_gen(7), device="cuda") * 2 - 1
    xb = xf.to(torch.bfloat16)
    d = api.make_desc(api.BF16, api.F32, rows, cols)
    out = _run(d, xb, torch.zeros(rows, device="cuda"))
    exp = u.oracle_reduce(d, _host(xb))
    assert u.fp_close(_host(out), exp).all(), u.worst_rel(_host(out), exp)
    # the same sums without splitting the rows (one team per row)
    d2 = api.make_desc(api.BF16, api.F32, rows, cols, plan_hint=api.PLAN_ROW_BLOCK)
    out2 = _run(d2, xb, torch.zeros(rows, device="cuda"))
    assert u.fp_close(_host(out2), exp).all()


# More than 2^31 elements through the plans whose addressing is newest: int8 data keep the
# memory at 2.3 GB and int64 sums are exact.  The oracle needs minutes for a sequential pass
# over this much, so the check is torch's own integer sums over the same device buffer, in
# pieces that stay below 2^31 elements (exact integer arithmetic, no tolerance); the same
# plans are held to the oracle at sizes it finishes in seconds in test_gpu_parity.py.
@pytest.mark.parametrize("rows,cols,apply", [
    (70_001, 32_768, api.ALONG_COLUMNS),     # wide rows cut in 64-lane pieces
    (17_400_001, 132, api.ALONG_COLUMNS),    # 9 lane-loads: whole rows packed into a workgroup
    (17_400_001, 132, api.ALONG_ROWS),       # 9 lane-loads with a tail: lane groups of 9
    (580_000_001, 4, api.ALONG_COLUMNS),     # rows shorter than a vector, read in groups
    (580_000_001, 4, api.ALONG_ROWS),        # several rows per 16-byte vector
])
def test_int8_sums_beyond_2g_elements(gpu, rows, cols, apply):
    import torch
    assert rows * cols > 2**31
    x = torch.randint(-128, 128, (rows * cols,), generator=_gen(rows % 1000 + cols),
                      device="cuda", dtype=torch.int8)
    n_out = rows if apply == api.ALONG_ROWS else cols
    d = api.make_desc(api.I8, api.I64, rows, cols, apply=apply)
    out = _run(d, x, torch.zeros(n_out, dtype=torch.int64, device="cuda"))
    m = x.view(rows, cols)
    step = max(1, (2**30) // cols)
    if apply == api.ALONG_ROWS:
        ref = torch.cat([m[r:r + step].sum(dim=1, dtype=torch.int64) for r in range(0, rows, step)])
    else:
        ref = torch.zeros(cols, dtype=torch.int64, device="cuda")
        for r in range(0, rows, step):
            ref += m[r:r + step].sum(dim=0, dtype=torch.int64)
    assert torch.equal(out, ref)


# The same for the one-pass mean / variance (f32, 9 GB) and for row normalisation (bf16,
# 4.5 GB in and out), against torch in f64 / f32 on the device.
def test_meanvar_beyond_2g_elements(gpu):
    import torch
    from raft_amd import device as dev
    rows, cols = 35_000_001, 64
    x = torch.randn(rows * cols, generator=_gen(11), device="cuda") * 2 + 3
    mean = torch.zeros(cols, device="cuda")
    var = torch.zeros(cols, device="cuda")
    dev.meanvar(api.F32, api.ROW_MAJOR, rows, cols, True, x, mean, var)
    torch.cuda.synchronize()
    m = x.view(rows, cols)
    ref_mean = torch.zeros(cols, dtype=torch.float64, device="cuda")
    step = 4_000_000
    for r in range(0, rows, step):
        ref_mean += m[r:r + step].sum(dim=0, dtype=torch.float64)
    ref_mean /= rows
    ref_m2 = torch.zeros(cols, dtype=torch.float64, device="cuda")
    for r in range(0, rows, step):
        ref_m2 += ((m[r:r + step].double() - ref_mean) ** 2).sum(dim=0)
    ref_var = ref_m2 / (rows - 1)
    assert u.fp_close(mean.cpu().numpy(), ref_mean.cpu().numpy()).all()
    assert u.fp_close(var.cpu().numpy(), ref_var.cpu().numpy()).all()


def test_row_normalize_beyond_2g_elements(gpu):
    import torch
    from raft_amd import device as dev
    rows, cols = 17_500_001, 128
    x = (torch.randn(rows * cols, generator=_gen(12), device="cuda") * 3).to(torch.bfloat16)
    out = torch.empty_like(x)
    d = api.make_desc(api.BF16, api.BF16, rows, cols, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT)
    rc = api.load().rmi_row_normalize(C.byref(d), x.data_ptr(), out.data_ptr(), 1e-8,
                                      dev.current_stream_ptr())
    assert rc == api.OK
    torch.cuda.synchronize()
    step = 2_000_000
    for r in (0, rows // 2, rows - step):          # three slices of 2M rows, last one included
        xs = x.view(rows, cols)[r:r + step].float()
        ref = xs / torch.linalg.vector_norm(xs, dim=1, keepdim=True)
        got = out.view(rows, cols)[r:r + step].float()
        assert torch.allclose(got, ref, rtol=2 ** -7, atol=1e-6)
    # unit rows everywhere (a checksum over all rows)
    n = torch.zeros(rows, device="cuda")
    for r in range(0, rows, step):
        n[r:r + step] = torch.linalg.vector_norm(out.view(rows, cols)[r:r + step].float(), dim=1)
    assert (n - 1).abs().max().item() < 2e-2
