"""The C ABI is stream-ordered, never synchronises and keeps no state between calls
(cpp/docs/source/developer_guide.md:20-24,421-431 asks that of every prim): calls from
several host threads on streams of their own give the same results as one call at a time,
and a call can be recorded into a HIP graph and replayed on new input contents."""
import ctypes as C
import threading

import numpy as np
import pytest

from raft_amd import _capi as api
from tests import _util as u

pytestmark = pytest.mark.gpu


def _cases():
    """(descriptor, numpy dtype, elements): one shape per plan kind, two of them with a
    second pass over a workspace."""
    kvp = dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX, init_f=-np.inf)
    return [
        (api.make_desc(api.F32, api.F32, 5000, 128, main_op=api.MAIN_SQ, final_op=api.FIN_SQRT),
         np.float32),                                                         # wave per row
        (api.make_desc(api.F32, api.F32, 3001, 33), np.float32),              # any lane count
        (api.make_desc(api.F32, api.F32, 20000, 100), np.float32),            # staged rows
        (api.make_desc(api.F32, api.KVP_I32_F32, 300, 9000, **kvp), np.float32),  # team per row
        (api.make_desc(api.F32, api.F32, 4, 300000), np.float32),             # split rows + fold
        (api.make_desc(api.F32, api.F32, 40000, 65, apply=api.ALONG_COLUMNS), np.float32),
        (api.make_desc(api.F32, api.F32, 50001, 3, apply=api.ALONG_COLUMNS), np.float32),
        (api.make_desc(api.I8, api.I64, 70000, 8), np.int8),                  # rows inside a vector
    ]


def _data(rng, dt, n):
    if dt == np.int8:
        return rng.integers(-128, 128, n, dtype=np.int8)
    return rng.uniform(-1, 1, n).astype(dt)


def _expect(desc, data):
    return u.oracle_reduce(desc, data)


def _check(desc, got_raw, exp, label):
    got = u.decode_out(desc.out_dtype, got_raw)
    if u.is_arg(desc):
        assert np.array_equal(got[0], exp[0]) and np.array_equal(got[1], exp[1]), label
    elif desc.out_dtype == api.I64:
        assert np.array_equal(got, exp), label
    else:
        assert u.fp_close(got, exp, u.OUT_TOL[desc.out_dtype]).all(), (label, u.worst_rel(got, exp))


def _launch(lib, desc, x, out, ws, stream_ptr):
    wsb = ws.numel() if ws is not None else 0
    rc = lib.rmi_reduce(C.byref(desc), x.data_ptr(), out.data_ptr(),
                        ws.data_ptr() if ws is not None else None, wsb, stream_ptr)
    assert rc == api.OK, api.status_string(rc)


def _buffers(torch, desc, data):
    odt = u.out_numpy_dtype(desc.out_dtype)
    x = torch.from_numpy(data.view(np.uint8)).cuda()
    out = torch.zeros(u.n_outputs(desc) * odt.itemsize, dtype=torch.uint8, device="cuda")
    wsb = api.load().rmi_reduce_workspace_bytes(C.byref(desc))
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda") if wsb else None
    return x, out, ws, odt


def test_threads_on_their_own_streams(gpu):
    """Four host threads, each with a stream and buffers of its own, issue every case ten
    times without synchronising in between; results are checked after one final sync."""
    import torch
    lib = api.load()
    cases = _cases()
    n_threads = 4
    work = []
    for t in range(n_threads):
        rng = np.random.default_rng(100 + t)
        mine = []
        for desc, dt in cases:
            data = _data(rng, dt, desc.n_rows * desc.n_cols)
            mine.append((desc, data, _expect(desc, data)) + _buffers(torch, desc, data))
        work.append(mine)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(n_threads)]
    errors = []

    def run(t):
        try:
            sp = streams[t].cuda_stream
            for _ in range(10):
                for desc, _, _, x, out, ws, _ in work[t]:
                    _launch(lib, desc, x, out, ws, sp)
        except Exception as e:  # noqa: BLE001 - reported by the main thread
            errors.append((t, e))

    threads = [threading.Thread(target=run, args=(t,)) for t in range(n_threads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for t in range(n_threads):
        for i, (desc, _, exp, _, out, _, odt) in enumerate(work[t]):
            _check(desc, out.cpu().numpy().view(odt), exp, f"thread {t} case {i}")


def test_graph_replay(gpu):
    """Every case recorded into one HIP graph on a side stream; the graph is replayed three
    times, the inputs are overwritten between replays, and every replay is checked."""
    import torch
    lib = api.load()
    cases = _cases()
    rng = np.random.default_rng(7)
    bufs = []
    for desc, dt in cases:
        data = _data(rng, dt, desc.n_rows * desc.n_cols)
        bufs.append((desc, dt) + _buffers(torch, desc, data))
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    # one eager pass on the side stream first (plans and device properties are cached by then)
    for desc, _, x, out, ws, _ in bufs:
        _launch(lib, desc, x, out, ws, side.cuda_stream)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        sp = torch.cuda.current_stream().cuda_stream
        for desc, _, x, out, ws, _ in bufs:
            _launch(lib, desc, x, out, ws, sp)
    for replay in range(3):
        expect = []
        for desc, dt, x, out, _, _ in bufs:
            data = _data(rng, dt, desc.n_rows * desc.n_cols)
            x.copy_(torch.from_numpy(data.view(np.uint8)))
            out.fill_(0x5A)
            expect.append(_expect(desc, data))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for i, ((desc, _, _, out, _, odt), exp) in enumerate(zip(bufs, expect)):
            _check(desc, out.cpu().numpy().view(odt), exp, f"replay {replay} case {i}")
