"""Shared helpers for the tests: the oracle binding, storage conversions, the
comparators and a one-call "run on the GPU through the C ABI" helper."""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

import numpy as np

from raft_amd import _capi as api

ROOT = Path(__file__).resolve().parent.parent
ORACLE_PATH = ROOT / "oracle" / "liboracle.so"

NP_OF = {api.I8: np.int8, api.U8: np.uint8, api.I32: np.int32, api.I64: np.int64,
         api.F16: np.float16, api.BF16: np.uint16, api.F32: np.float32, api.F64: np.float64}

KVP_NP = {
    api.KVP_I32_F32: np.dtype([("key", np.int32), ("value", np.float32)], align=True),
    api.KVP_I32_F64: np.dtype([("key", np.int32), ("value", np.float64)], align=True),
    api.KVP_I64_F32: np.dtype([("key", np.int64), ("value", np.float32)], align=True),
    api.KVP_I64_F64: np.dtype([("key", np.int64), ("value", np.float64)], align=True),
}
assert [KVP_NP[k].itemsize for k in sorted(KVP_NP)] == [8, 16, 16, 16]

_oracle = None


def load_oracle() -> C.CDLL:
    global _oracle
    if _oracle is None:
        if not ORACLE_PATH.exists():
            raise RuntimeError(f"{ORACLE_PATH} is not built; run `python -m raft_amd.build`")
        lib = C.CDLL(str(ORACLE_PATH))
        lib.orc_reduce.restype = C.c_int
        lib.orc_reduce.argtypes = [C.POINTER(api.ReduceDesc), C.c_void_p, C.c_void_p, C.c_void_p,
                                   C.c_void_p, C.c_void_p, C.c_void_p]
        lib.orc_reduce_typed.restype = C.c_int
        lib.orc_reduce_typed.argtypes = [C.POINTER(api.ReduceDesc), C.c_void_p, C.c_void_p,
                                         C.c_void_p, C.c_int]
        lib.orc_max_threads.restype = C.c_int
        lib.orc_row_normalize.restype = C.c_int
        lib.orc_row_normalize.argtypes = [C.POINTER(api.ReduceDesc), C.c_void_p, C.c_void_p,
                                          C.c_double]
        lib.orc_meanvar.restype = C.c_int
        lib.orc_meanvar.argtypes = [C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int, C.c_void_p,
                                    C.c_void_p, C.c_void_p]
        lib.orc_cov.restype = C.c_int
        lib.orc_cov.argtypes = [C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int, C.c_void_p,
                                C.c_void_p, C.c_void_p, C.c_void_p]
        for name in ("orc_f32_to_bf16", "orc_bf16_to_f32", "orc_f32_to_f16", "orc_f16_to_f32"):
            getattr(lib, name).restype = None
            getattr(lib, name).argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        _oracle = lib
    return _oracle


def to_bf16(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    load_oracle().orc_f32_to_bf16(x.ctypes.data, out.ctypes.data, x.size)
    return out


def from_bf16(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    load_oracle().orc_bf16_to_f32(x.ctypes.data, out.ctypes.data, x.size)
    return out


def n_outputs(desc: api.ReduceDesc) -> int:
    return desc.n_rows if desc.apply == api.ALONG_ROWS else desc.n_cols


def is_arg(desc) -> bool:
    return desc.reduce_op in (api.RED_ARGMAX, api.RED_ARGMIN)


def oracle_reduce(desc: api.ReduceDesc, data: np.ndarray, *, old=None, aux=None):
    """Sequential fp64/int64 oracle.  Returns a float64 array (floating outputs), an
    int64 array (integer outputs) or (keys int64, values float64) for arg reductions.
    `old`: previous output values when desc.inplace (float64 / int64 / (keys, values));
    `aux`: float64 per-output vector for the VAR/STDDEV epilogue."""
    lib = load_oracle()
    n = n_outputs(desc)
    data = np.ascontiguousarray(data)
    out_f = np.zeros(n, dtype=np.float64)
    out_i = np.zeros(n, dtype=np.int64)
    old_f = old_i = None
    if desc.inplace:
        if is_arg(desc):
            old_i = np.ascontiguousarray(old[0], dtype=np.int64)
            old_f = np.ascontiguousarray(old[1], dtype=np.float64)
        elif desc.out_dtype in (api.I32, api.I64):
            old_i = np.ascontiguousarray(old, dtype=np.int64)
        else:
            old_f = np.ascontiguousarray(old, dtype=np.float64)
    aux_f = np.ascontiguousarray(aux, dtype=np.float64) if aux is not None else None
    ptr = lambda a: a.ctypes.data if a is not None else None
    d = api.ReduceDesc.from_buffer_copy(desc)
    d.final_aux = None
    rc = lib.orc_reduce(C.byref(d), ptr(data), ptr(old_f), ptr(old_i), ptr(aux_f), ptr(out_f),
                        ptr(out_i))
    assert rc == api.OK, f"oracle refused the descriptor: status {rc}"
    if is_arg(desc):
        return out_i, out_f
    if desc.out_dtype in (api.I32, api.I64):
        return out_i
    return out_f


def oracle_typed(desc: api.ReduceDesc, data: np.ndarray, out: np.ndarray, aux=None, threads=0):
    """OpenMP implementation in the output's own arithmetic; writes into `out`."""
    lib = load_oracle()
    d = api.ReduceDesc.from_buffer_copy(desc)
    d.final_aux = None
    rc = lib.orc_reduce_typed(C.byref(d), data.ctypes.data, out.ctypes.data,
                              aux.ctypes.data if aux is not None else None, threads)
    assert rc == api.OK, f"typed oracle refused the descriptor: status {rc}"
    return out


# Comparator of the reference's tests (cpp/tests/test_utils.h:32-45): pass if the
# absolute OR the relative difference is within eps.
def approx_ok(actual, expected, eps):
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    diff = np.abs(actual - expected)
    m = np.maximum(np.abs(actual), np.abs(expected))
    with np.errstate(divide="ignore", invalid="ignore"):
        ratio = np.where(m > 0, diff / m, 0.0)
    same_special = (actual == expected) | (np.isnan(actual) & np.isnan(expected))
    return same_special | (diff <= eps) | (ratio <= eps)


# The bar of this build for floating results against the fp64 oracle:
# |x - o| <= 1e-5*|o|, or <= 1e-5 absolute where |o| < 1.
FP_TOL = 1e-5
OUT_TOL = {api.F32: 1e-5, api.F64: 1e-5}
# 16-bit outputs have no tolerance: the library rounds its f64 result once, so an output must be
# the correctly rounded oracle value or the 16-bit number next to it (ulp16_ok below).


def _ord16(bits):
    """uint16 sign-magnitude storage bits -> integers ordered like the values (+-0 -> 0)."""
    b = np.asarray(bits).astype(np.int32)
    return np.where(b & 0x8000, -(b & 0x7FFF), b)


def _bits16(o):
    o = np.asarray(o, dtype=np.int32)
    return np.where(o < 0, (-o) | 0x8000, o).astype(np.uint16)


def round_to_16(out_dtype, values):
    """float64 values -> storage bits of the nearest f16 / bf16 number (ties to even)."""
    v = np.asarray(values, dtype=np.float64)
    if out_dtype == api.F16:
        with np.errstate(over="ignore"):
            return v.astype(np.float16).view(np.uint16)
    # bf16: round through f32, then repair the rare double rounding by picking, among the
    # result and its two neighbours, the one strictly nearest to the f64 value
    with np.errstate(over="ignore"):
        b0 = to_bf16(v.astype(np.float32))
    o0 = _ord16(b0)
    best, bestd = o0.copy(), np.abs(from_bf16(b0).astype(np.float64) - v)
    for step in (-1, 1):
        c = o0 + step
        with np.errstate(invalid="ignore"):
            d = np.abs(from_bf16(_bits16(c)).astype(np.float64) - v)
        take = np.isfinite(d) & (d < bestd)
        best, bestd = np.where(take, c, best), np.where(take, d, bestd)
    return np.where(np.isfinite(v), _bits16(best), b0).astype(np.uint16)


def ulp16_ok(out_dtype, got_bits, expected_f64, ulps=1):
    """True where a 16-bit output is within `ulps` representable numbers of the correctly
    rounded expected value (NaN matches NaN, infinities match themselves)."""
    got_bits = np.asarray(got_bits).view(np.uint16)
    want = round_to_16(out_dtype, expected_f64)
    gf = got_bits.view(np.float16).astype(np.float64) if out_dtype == api.F16 else \
        from_bf16(got_bits).astype(np.float64)
    nan = np.isnan(np.asarray(expected_f64, dtype=np.float64))
    return np.where(nan, np.isnan(gf), np.abs(_ord16(got_bits) - _ord16(want)) <= ulps)


def fp_close(actual, expected, tol=FP_TOL):
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    with np.errstate(invalid="ignore"):
        diff = np.abs(actual - expected)
        bound = tol * np.maximum(np.abs(expected), 1.0)
    same_special = (actual == expected) | (np.isnan(actual) & np.isnan(expected))
    return same_special | (diff <= bound)


def worst_rel(actual, expected):
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    d = np.abs(actual - expected) / np.maximum(np.abs(expected), 1.0)
    d = np.where(np.isfinite(d), d, 0.0)
    return float(d.max()) if d.size else 0.0


def out_numpy_dtype(out_dtype):
    return KVP_NP[out_dtype] if out_dtype in KVP_NP else np.dtype(NP_OF[out_dtype])


def decode_out(out_dtype, raw: np.ndarray):
    """Raw output array -> float64 / int64 / (keys, values) in the oracle's form."""
    if out_dtype in KVP_NP:
        return raw["key"].astype(np.int64), raw["value"].astype(np.float64)
    if out_dtype == api.BF16:
        return from_bf16(raw).astype(np.float64)
    if out_dtype in (api.I32, api.I64):
        return raw.astype(np.int64)
    return raw.astype(np.float64)


def encode_out(out_dtype, values):
    """Oracle-form values -> raw array of the output dtype (for inplace seeds, aux)."""
    if out_dtype in KVP_NP:
        raw = np.zeros(len(values[0]), dtype=KVP_NP[out_dtype])
        raw["key"] = values[0]
        raw["value"] = values[1]
        return raw
    if out_dtype == api.BF16:
        return to_bf16(np.asarray(values, dtype=np.float32))
    return np.asarray(values).astype(NP_OF[out_dtype])


def gpu_reduce(desc: api.ReduceDesc, data: np.ndarray, *, old_raw=None, aux_raw=None,
               misalign_elems: int = 0, workspace=None):
    """Upload `data`, run rmi_reduce through the C ABI on cuda:0, return the raw output
    array (numpy, output dtype).  `old_raw` seeds the output buffer (inplace);
    `aux_raw` is uploaded and passed as final_aux; `misalign_elems` shifts the input's
    device address by that many elements to exercise the element-wise load path;
    `workspace` is a device tensor to use instead of a fresh one (a shared, zeroed
    workspace for descriptors that carry RMI_FLAG_WORKSPACE_ZEROED)."""
    import torch
    from raft_amd import device as dev

    n = n_outputs(desc)
    odt = out_numpy_dtype(desc.out_dtype)
    data = np.ascontiguousarray(data)
    flat = torch.from_numpy(data.reshape(-1).view(np.uint8))
    es = data.dtype.itemsize
    pad = misalign_elems * es
    buf = torch.empty(flat.numel() + pad + 16, dtype=torch.uint8, device="cuda")
    buf[pad:pad + flat.numel()].copy_(flat)
    out = torch.zeros(max(n, 1) * odt.itemsize, dtype=torch.uint8, device="cuda")
    if old_raw is not None:
        out[: n * odt.itemsize].copy_(torch.from_numpy(
            np.ascontiguousarray(old_raw).view(np.uint8).reshape(-1)))
    aux_t = None
    d = api.ReduceDesc.from_buffer_copy(desc)
    if aux_raw is not None:
        aux_t = torch.from_numpy(np.ascontiguousarray(aux_raw).view(np.uint8).reshape(-1)).cuda()
        d.final_aux = aux_t.data_ptr()
    dev.reduce(d, buf, out, workspace, in_ptr=buf.data_ptr() + pad)
    torch.cuda.synchronize()
    raw = out.cpu().numpy()[: n * odt.itemsize].view(odt).copy()
    return raw


def check_against_oracle(desc, data, *, old_raw=None, aux_raw=None, misalign_elems=0,
                         tol=None, label=""):
    """GPU result vs the fp64 oracle on the same input, at the build's bar: exact for
    integers and arg-reductions, FP_TOL (or the output type's own rounding) for floats."""
    got_raw = gpu_reduce(desc, data, old_raw=old_raw, aux_raw=aux_raw,
                         misalign_elems=misalign_elems)
    got = decode_out(desc.out_dtype, got_raw)
    old = decode_out(desc.out_dtype, old_raw) if old_raw is not None else None
    aux = decode_out(desc.out_dtype, aux_raw) if aux_raw is not None else None
    exp = oracle_reduce(desc, data, old=old, aux=aux)
    if is_arg(desc):
        ek, ev = exp
        if desc.final_op == api.FIN_KEY:
            assert np.array_equal(got, ek), f"{label}: arg keys differ"
        else:
            gk, gv = got
            assert np.array_equal(gk, ek), (
                f"{label}: arg keys differ at {np.flatnonzero(gk != ek)[:8]}")
            assert np.array_equal(gv, ev), f"{label}: arg values differ"
    elif desc.out_dtype in (api.I32, api.I64):
        if desc.out_dtype == api.I32:
            exp = exp.astype(np.int32).astype(np.int64)
        assert np.array_equal(got, exp), (
            f"{label}: integer results differ at {np.flatnonzero(got != exp)[:8]}")
    elif desc.out_dtype in (api.F16, api.BF16) and tol is None:
        ok = ulp16_ok(desc.out_dtype, got_raw, exp)
        assert ok.all(), (f"{label}: {np.count_nonzero(~ok)} of {ok.size} 16-bit outputs are more "
                          f"than one ulp from the rounded oracle value: first bad "
                          f"{np.flatnonzero(~ok)[:5]} got {got[~ok][:5]} want {exp[~ok][:5]}")
    else:
        t = tol if tol is not None else OUT_TOL[desc.out_dtype]
        ok = fp_close(got, exp, t)
        assert ok.all(), (f"{label}: {np.count_nonzero(~ok)} of {ok.size} outputs beyond {t}: "
                          f"worst rel {worst_rel(got, exp):.3e}, first bad "
                          f"{np.flatnonzero(~ok)[:5]} got {got[~ok][:5]} want {exp[~ok][:5]}")
    return got_raw


def golden():
    """The reference's known-answer vectors (tests/golden/reference_fixtures.json)."""
    import json
    global _golden
    try:
        return _golden
    except NameError:
        pass
    with open(os.path.join(os.path.dirname(__file__), "golden", "reference_fixtures.json")) as f:
        _golden = json.load(f)
    return _golden


LAYOUT_AXIS = {"row_major/along_rows": (api.ROW_MAJOR, api.ALONG_ROWS),
               "row_major/along_columns": (api.ROW_MAJOR, api.ALONG_COLUMNS),
               "col_major/along_rows": (api.COL_MAJOR, api.ALONG_ROWS),
               "col_major/along_columns": (api.COL_MAJOR, api.ALONG_COLUMNS)}
