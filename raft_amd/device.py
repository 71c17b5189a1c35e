"""Pass torch device tensors through the C ABI (device memory and streams only).

torch provides allocation, the current HIP stream and events; every reduction
is computed by libraft_amd.so.  A missing library or a non-OK status raises.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _capi as api


class RmiError(RuntimeError):
    def __init__(self, code: int, where: str):
        super().__init__(f"{where}: {api.status_string(code)} (status {code})")
        self.code = code


def current_stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def workspace_for(desc: api.ReduceDesc, device="cuda") -> torch.Tensor | None:
    n = api.load().rmi_reduce_workspace_bytes(C.byref(desc))
    if n == 0:
        return None
    return torch.empty(n, dtype=torch.uint8, device=device)


def reduce(desc: api.ReduceDesc, inp: torch.Tensor, out: torch.Tensor,
           workspace: torch.Tensor | None = None, *, in_ptr: int | None = None,
           out_ptr: int | None = None) -> None:
    """Run rmi_reduce on the current torch stream.  `inp` / `out` are device tensors
    whose storage is interpreted according to the descriptor's dtypes."""
    lib = api.load()
    if workspace is None:
        workspace = workspace_for(desc, inp.device if inp is not None else out.device)
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    ip = in_ptr if in_ptr is not None else (inp.data_ptr() if inp is not None else None)
    op = out_ptr if out_ptr is not None else out.data_ptr()
    rc = lib.rmi_reduce(C.byref(desc), ip, op, ws_ptr, ws_bytes, current_stream_ptr())
    if rc != api.OK:
        raise RmiError(rc, "rmi_reduce")


def map_reduce(desc: api.ReduceDesc, length: int, inp: torch.Tensor, out: torch.Tensor) -> None:
    lib = api.load()
    n = lib.rmi_map_reduce_workspace_bytes(C.byref(desc), length)
    ws = torch.empty(max(n, 1), dtype=torch.uint8, device=inp.device)
    rc = lib.rmi_map_reduce(C.byref(desc), length, inp.data_ptr(), out.data_ptr(),
                            ws.data_ptr(), n, current_stream_ptr())
    if rc != api.OK:
        raise RmiError(rc, "rmi_map_reduce")


def meanvar(dtype: int, layout: int, n_rows: int, n_cols: int, sample: bool,
            data: torch.Tensor, mean: torch.Tensor, var: torch.Tensor) -> None:
    """Run rmi_meanvar on the current torch stream."""
    lib = api.load()
    n = lib.rmi_meanvar_workspace_bytes(dtype, layout, n_rows, n_cols)
    ws = torch.empty(n, dtype=torch.uint8, device=data.device) if n else None
    rc = lib.rmi_meanvar(dtype, layout, n_rows, n_cols, 1 if sample else 0, data.data_ptr(),
                         mean.data_ptr(), var.data_ptr(), ws.data_ptr() if n else None, n,
                         current_stream_ptr())
    if rc != api.OK:
        raise RmiError(rc, "rmi_meanvar")


def cov(dtype: int, layout: int, n_rows: int, n_cols: int, sample: bool, data: torch.Tensor,
        mu: torch.Tensor | None, covar: torch.Tensor, *, center: bool = False) -> None:
    """Run rmi_cov on the current torch stream; with `center` the call leaves x - mu in `data`."""
    lib = api.load()
    n = lib.rmi_cov_workspace_bytes(dtype, layout, n_rows, n_cols)
    ws = torch.empty(max(n, 16), dtype=torch.uint8, device=covar.device)
    rc = lib.rmi_cov(dtype, layout, n_rows, n_cols, 1 if sample else 0,
                     api.COV_CENTER_DATA if center else 0,
                     data.data_ptr() if data is not None else None,
                     mu.data_ptr() if mu is not None else None, covar.data_ptr(), ws.data_ptr(), n,
                     current_stream_ptr())
    if rc != api.OK:
        raise RmiError(rc, "rmi_cov")
