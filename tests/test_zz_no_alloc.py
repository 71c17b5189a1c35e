"""rmi_reduce_noalloc: the entry point that allocates nothing (partials of two-pass plans go
to the library's static device buffer) against rmi_reduce with a caller's workspace, through
the C ABI.  Results must be identical bit for bit; two calls in a row share the buffer, the
second with a smaller input."""
import ctypes as C

import numpy as np
import pytest

from raft_amd import _capi as api

pytestmark = pytest.mark.gpu


def _both(desc, x, out_dtype_bytes, n_out):
    """Run rmi_reduce (own workspace) and rmi_reduce_noalloc on the same device input."""
    import torch
    lib = api.load()
    sptr = torch.cuda.current_stream().cuda_stream
    nws = lib.rmi_reduce_workspace_bytes(C.byref(desc))
    ws = torch.empty(max(nws, 16), dtype=torch.uint8, device="cuda")
    a = torch.full((n_out * out_dtype_bytes,), 0x5A, dtype=torch.uint8, device="cuda")
    b = torch.full((n_out * out_dtype_bytes,), 0xA5, dtype=torch.uint8, device="cuda")
    rc = lib.rmi_reduce(C.byref(desc), x.data_ptr(), a.data_ptr(), ws.data_ptr(), nws, sptr)
    assert rc == api.OK, api.status_string(rc)
    # "allocates nothing" is held to the device's own count of free memory, which sees any
    # allocation of any library (torch's allocator counter would only see torch's): the first
    # call on this device looked the buffer's address up, so from here on nothing may move
    rc = lib.rmi_reduce_noalloc(C.byref(desc), x.data_ptr(), b.data_ptr(), sptr)
    assert rc == api.OK, api.status_string(rc)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    before = torch.cuda.memory_allocated()
    for _ in range(3):
        rc = lib.rmi_reduce_noalloc(C.byref(desc), x.data_ptr(), b.data_ptr(), sptr)
        assert rc == api.OK, api.status_string(rc)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
    assert torch.cuda.memory_allocated() == before
    return a.cpu().numpy(), b.cpu().numpy(), nws


# (in dtype, out dtype, out bytes, kwargs, [(rows, cols) first call, (rows, cols) second, smaller])
CASES = [
    # split rows (two passes: partials per row chunk)
    (api.BF16, api.F32, 4, {}, [(8, 1 << 20), (3, 300_000)]),
    (api.F32, api.F32, 4, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT), [(4, 2_000_003), (2, 500_001)]),
    (api.F64, api.F64, 8, {}, [(2, 1_000_000), (1, 200_000)]),
    (api.I8, api.I64, 8, {}, [(5, 4_000_000), (5, 1_000_000)]),
    (api.F32, api.KVP_I32_F32, 8, dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX,
                                       init_f=-np.inf), [(3, 1_000_000), (2, 400_000)]),
    # column reductions (two passes: partials per block of rows)
    (api.F32, api.F32, 4, dict(apply=api.ALONG_COLUMNS), [(2_000_000, 64), (100_000, 64)]),
    (api.F32, api.F32, 4, dict(apply=api.ALONG_COLUMNS, main_op=api.MAIN_SQ), [(300_000, 3), (50_000, 3)]),
    (api.I8, api.I64, 8, dict(apply=api.ALONG_COLUMNS), [(1_000_000, 130), (20_000, 130)]),
    (api.F64, api.F64, 8, dict(apply=api.ALONG_COLUMNS, reduce_op=api.RED_MAX, init_f=-np.inf),
     [(200_000, 1000), (5_000, 1000)]),
    # single-pass plans take the same entry point and need no scratch
    (api.F32, api.F32, 4, {}, [(10000, 256), (100, 256)]),
]


@pytest.mark.parametrize("in_dt,out_dt,out_bytes,kw,shapes", CASES)
def test_noalloc_matches_rmi_reduce(gpu, in_dt, out_dt, out_bytes, kw, shapes):
    import torch
    tdt = {api.BF16: torch.bfloat16, api.F32: torch.float32, api.F64: torch.float64,
           api.I8: torch.int8}[in_dt]
    g = torch.Generator(device="cuda")
    g.manual_seed(shapes[0][0] + shapes[0][1])
    two_pass = 0
    for rows, cols in shapes:          # two calls in a row, the second with a smaller input
        n = rows * cols
        if in_dt == api.I8:
            x = torch.randint(-128, 128, (n,), generator=g, device="cuda", dtype=torch.int8)
        else:
            x = torch.randn(n, generator=g, device="cuda", dtype=torch.float32).to(tdt)
        d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
        n_out = rows if d.apply == api.ALONG_ROWS else cols
        a, b, nws = _both(d, x, out_bytes, n_out)
        assert np.array_equal(a, b), (rows, cols)
        two_pass += nws > 0
    if shapes[0] != (10000, 256):
        assert two_pass == len(shapes), "these shapes are meant to use the scratch buffer"


def test_noalloc_refuses_plans_beyond_its_buffer(gpu):
    import torch
    lib = api.load()
    # arg-max with 64-bit keys down 500 columns: 768 blocks of rows x 16-byte partials > 4 MiB
    rows, cols = 20_000, 500
    d = api.make_desc(api.F32, api.KVP_I64_F32, rows, cols, apply=api.ALONG_COLUMNS,
                      main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, init_f=-np.inf)
    need = lib.rmi_reduce_workspace_bytes(C.byref(d))
    assert need > api.NOALLOC_SCRATCH_BYTES
    x = torch.zeros(rows * cols, device="cuda")
    out = torch.full((cols * 4,), 7.0, device="cuda")
    rc = lib.rmi_reduce_noalloc(C.byref(d), x.data_ptr(), out.data_ptr(),
                                torch.cuda.current_stream().cuda_stream)
    assert rc == api.ERR_SCRATCH_LIMIT
    assert "scratch" in api.status_string(rc)
    torch.cuda.synchronize()
    assert bool((out == 7.0).all()), "nothing may be launched"


def test_noalloc_passes_over_plans_with_large_partials(gpu):
    """Column sums of wide rows: rmi_reduce streams whole rows with one set of partials per
    CU, more than the static buffer holds at this width; the entry point that allocates nothing
    takes the layout with fewer partials instead of refusing the call."""
    import torch
    lib = api.load()
    rows, cols = 16384, 4097
    d = api.make_desc(api.F32, api.F32, rows, cols, apply=api.ALONG_COLUMNS)
    assert lib.rmi_reduce_workspace_bytes(C.byref(d)) > api.NOALLOC_SCRATCH_BYTES
    x = torch.randn(rows * cols, device="cuda")
    a, b, _ = _both(d, x, 4, cols)
    a, b = a.view(np.float32), b.view(np.float32)
    # both accumulate in fp64 and round once; the partial sums are grouped differently
    assert np.allclose(a, b, rtol=3e-7, atol=0), np.abs(a - b).max()
    want = x.view(rows, cols).sum(dim=0, dtype=torch.float64).cpu().numpy()
    assert np.allclose(b, want, rtol=1e-6, atol=1e-6)
    # the library's own flag bit is refused from callers
    d.flags = 1 << 30
    assert lib.rmi_reduce_workspace_bytes(C.byref(d)) == 0
    out = torch.zeros(cols, device="cuda")
    sptr = torch.cuda.current_stream().cuda_stream
    assert lib.rmi_reduce_noalloc(C.byref(d), x.data_ptr(), out.data_ptr(), sptr) == api.ERR_BAD_ENUM
    assert lib.rmi_reduce(C.byref(d), x.data_ptr(), out.data_ptr(), None, 0, sptr) == api.ERR_BAD_ENUM


def test_noalloc_under_graph_capture(gpu):
    """The caller this entry point is for: a captured stream, replayed over new inputs."""
    import torch
    lib = api.load()
    rows, cols = 4, 1_000_000
    d = api.make_desc(api.F32, api.F32, rows, cols)
    x = torch.randn(rows * cols, device="cuda")
    out = torch.zeros(rows, device="cuda")
    ref = torch.zeros(rows, device="cuda")
    nws = lib.rmi_reduce_workspace_bytes(C.byref(d))
    assert nws > 0
    ws = torch.empty(nws, dtype=torch.uint8, device="cuda")
    # the device's first call happens outside capture (it looks up the buffer's address)
    rc = lib.rmi_reduce_noalloc(C.byref(d), x.data_ptr(), out.data_ptr(),
                                torch.cuda.current_stream().cuda_stream)
    assert rc == api.OK
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.rmi_reduce_noalloc(C.byref(d), x.data_ptr(), out.data_ptr(), side.cuda_stream)
            assert rc == api.OK
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        x.normal_()
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        rc = lib.rmi_reduce(C.byref(d), x.data_ptr(), ref.data_ptr(), ws.data_ptr(), nws,
                            torch.cuda.current_stream().cuda_stream)
        assert rc == api.OK
        torch.cuda.synchronize()
        assert torch.equal(out, ref), rep


def test_noalloc_splits_rows_in_one_launch(gpu):
    """The static buffer's ticket words are zero from load time on, so rows split over several
    workgroups take the single-launch plan here; bit for bit the two-launch result."""
    import torch
    lib = api.load()
    d = api.make_desc(api.BF16, api.F32, 8, 4194304, flags=api.FLAG_WORKSPACE_ZEROED)
    assert api.plan_query(d).passes == 1
    d.flags = 0
    assert api.plan_query(d).passes == 2
    x = torch.randn(8 * 4194304, device="cuda").to(torch.bfloat16)
    for rep in range(3):
        a, b, nws = _both(d, x, 4, 8)
        assert nws > 0 and np.array_equal(a, b), rep
