"""ctypes view of the C ABI in include/rmi_reduce.h.

Used by the tests and the benchmark to reach the library exactly the way a
foreign-function caller would: plain pointers, sizes and a POD descriptor.
There is no fallback: if the shared library is missing this raises.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libraft_amd.so"

# rmi_status
OK, ERR_NULL, ERR_BAD_ENUM, ERR_BAD_SHAPE, ERR_UNSUPPORTED, ERR_WORKSPACE, ERR_ALIGNMENT, \
    ERR_LAUNCH, ERR_NO_DEVICE, ERR_SCRATCH_LIMIT = range(10)
ABI_VERSION = 3
NOALLOC_SCRATCH_BYTES = 4 << 20
FLAG_WORKSPACE_ZEROED = 1
COV_CENTER_DATA = 1
WORKSPACE_TICKET_BYTES = 65536

# rmi_dtype
I8, U8, I32, I64, F16, BF16, F32, F64, KVP_I32_F32, KVP_I32_F64, KVP_I64_F32, KVP_I64_F64 = range(12)
DTYPE_SIZE = {I8: 1, U8: 1, I32: 4, I64: 8, F16: 2, BF16: 2, F32: 4, F64: 8,
              KVP_I32_F32: 8, KVP_I32_F64: 16, KVP_I64_F32: 16, KVP_I64_F64: 16}
DTYPE_NAME = {I8: "i8", U8: "u8", I32: "i32", I64: "i64", F16: "f16", BF16: "bf16", F32: "f32",
              F64: "f64", KVP_I32_F32: "kvp<i32,f32>", KVP_I32_F64: "kvp<i32,f64>",
              KVP_I64_F32: "kvp<i64,f32>", KVP_I64_F64: "kvp<i64,f64>"}

ROW_MAJOR, COL_MAJOR = 0, 1
ALONG_ROWS, ALONG_COLUMNS = 0, 1

MAIN_IDENTITY, MAIN_SQ, MAIN_ABS, MAIN_NZ, MAIN_KVP = range(5)
RED_ADD, RED_MAX, RED_MIN, RED_ARGMAX, RED_ARGMIN = range(5)
(FIN_IDENTITY, FIN_SQRT, FIN_ABS, FIN_SQ, FIN_MUL_CONST, FIN_DIV_CONST, FIN_ADD_CONST,
 FIN_SUB_CONST, FIN_VAR_FROM_SUMSQ, FIN_STDDEV_FROM_SUMSQ, FIN_KEY) = range(11)

(PLAN_AUTO, PLAN_ROW_LANES, PLAN_ROW_WAVE, PLAN_ROW_BLOCK, PLAN_ROW_SPLIT, PLAN_COL_TILE,
 PLAN_EMPTY) = range(7)
PLAN_NAME = {PLAN_AUTO: "auto", PLAN_ROW_LANES: "row_lanes", PLAN_ROW_WAVE: "row_wave",
             PLAN_ROW_BLOCK: "row_block", PLAN_ROW_SPLIT: "row_split", PLAN_COL_TILE: "col_tile",
             PLAN_EMPTY: "empty"}


class Scalar(C.Structure):
    _fields_ = [("f", C.c_double), ("i", C.c_int64)]


class ReduceDesc(C.Structure):
    _fields_ = [
        ("in_dtype", C.c_int32), ("out_dtype", C.c_int32),
        ("layout", C.c_int32), ("apply", C.c_int32),
        ("n_rows", C.c_int64), ("n_cols", C.c_int64),
        ("main_op", C.c_int32), ("reduce_op", C.c_int32),
        ("final_op", C.c_int32), ("inplace", C.c_int32),
        ("init", Scalar),
        ("final_scalar", C.c_double), ("final_scalar2", C.c_double),
        ("final_aux", C.c_void_p),
        ("plan_hint", C.c_int32), ("flags", C.c_int32),
    ]


class Plan(C.Structure):
    _fields_ = [
        ("kind", C.c_int32), ("vec_bytes", C.c_int32), ("lanes_per_row", C.c_int32),
        ("blocks_per_out", C.c_int32), ("block_threads", C.c_int32), ("passes", C.c_int32),
        ("grid_blocks", C.c_int64), ("n_outputs", C.c_int64), ("reduce_len", C.c_int64),
        ("workspace_bytes", C.c_size_t),
    ]


# every symbol include/rmi_reduce.h declares: name -> (restype, argtypes)
SYMBOLS = {
    "rmi_abi_version": (C.c_int, []),
    "rmi_status_string": (C.c_char_p, [C.c_int]),
    "rmi_dtype_size": (C.c_size_t, [C.c_int]),
    "rmi_plan_query": (C.c_int, [C.POINTER(ReduceDesc), C.POINTER(Plan)]),
    "rmi_reduce_workspace_bytes": (C.c_size_t, [C.POINTER(ReduceDesc)]),
    "rmi_reduce": (C.c_int, [C.POINTER(ReduceDesc), C.c_void_p, C.c_void_p, C.c_void_p,
                             C.c_size_t, C.c_void_p]),
    "rmi_reduce_noalloc": (C.c_int, [C.POINTER(ReduceDesc), C.c_void_p, C.c_void_p, C.c_void_p]),
    "rmi_workspace_reset": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p]),
    "rmi_noalloc_reset": (C.c_int, [C.c_void_p]),
    "rmi_map_reduce_workspace_bytes": (C.c_size_t, [C.POINTER(ReduceDesc), C.c_int64]),
    "rmi_row_normalize": (C.c_int, [C.POINTER(ReduceDesc), C.c_void_p, C.c_void_p, C.c_double,
                                    C.c_void_p]),
    "rmi_map_reduce": (C.c_int, [C.POINTER(ReduceDesc), C.c_int64, C.c_void_p, C.c_void_p,
                                 C.c_void_p, C.c_size_t, C.c_void_p]),
    "rmi_meanvar_workspace_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int64, C.c_int64]),
    "rmi_meanvar": (C.c_int, [C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int, C.c_void_p,
                              C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "rmi_cov_workspace_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int64, C.c_int64]),
    "rmi_cov": (C.c_int, [C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_void_p,
                          C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
}

_lib = None


def load() -> C.CDLL:
    """Load libraft_amd.so and bind every declared symbol; raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is not built; run `python -m raft_amd.build` (there is no CPU fallback)")
    lib = C.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def status_string(code: int) -> str:
    return load().rmi_status_string(code).decode()


def make_desc(in_dtype, out_dtype, n_rows, n_cols, *, layout=ROW_MAJOR, apply=ALONG_ROWS,
              main_op=MAIN_IDENTITY, reduce_op=RED_ADD, final_op=FIN_IDENTITY, inplace=False,
              init_f=0.0, init_i=0, final_scalar=0.0, final_scalar2=0.0, final_aux=None,
              plan_hint=PLAN_AUTO, flags=0) -> ReduceDesc:
    d = ReduceDesc()
    d.in_dtype, d.out_dtype = in_dtype, out_dtype
    d.layout, d.apply = layout, apply
    d.n_rows, d.n_cols = n_rows, n_cols
    d.main_op, d.reduce_op, d.final_op = main_op, reduce_op, final_op
    d.inplace = 1 if inplace else 0
    d.init = Scalar(float(init_f), int(init_i))
    d.final_scalar, d.final_scalar2 = float(final_scalar), float(final_scalar2)
    d.final_aux = final_aux
    d.plan_hint = plan_hint
    d.flags = flags
    return d


def plan_query(desc: ReduceDesc) -> Plan:
    p = Plan()
    rc = load().rmi_plan_query(C.byref(desc), C.byref(p))
    if rc != OK:
        raise ValueError(f"rmi_plan_query: {status_string(rc)}")
    return p
