"""CPU-side checks of the C ABI: the library loads, exports every symbol that
include/rmi_reduce.h declares, validates descriptors and plans the benchmark shapes
as designed.  No kernel is launched here."""
import ctypes as C
import re
from pathlib import Path

import pytest

from raft_amd import _capi as api

ROOT = Path(__file__).resolve().parent.parent


def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "rmi_reduce.h").read_text()
    declared = set(re.findall(r"RMI_API\s+[\w\s\*]+?\b(rmi_\w+)\s*\(", header))
    assert declared, "no RMI_API declarations found"
    assert declared == set(api.SYMBOLS), (declared ^ set(api.SYMBOLS))
    lib = api.load()
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.rmi_abi_version() == api.ABI_VERSION


def test_struct_layouts_match_the_header(tmp_path):
    # the header must compile as plain C, and the ctypes mirrors must have the sizes and
    # field offsets the C compiler gives the two PODs
    import subprocess
    fields_d = [n for n, _ in api.ReduceDesc._fields_]
    fields_p = [n for n, _ in api.Plan._fields_]
    src = tmp_path / "layout.c"
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "rmi_reduce.h"', 'int main(void){',
             'printf("%zu %zu\\n", sizeof(rmi_reduce_desc), sizeof(rmi_plan));']
    lines += [f'printf("%zu\\n", offsetof(rmi_reduce_desc, {f}));' for f in fields_d]
    lines += [f'printf("%zu\\n", offsetof(rmi_plan, {f}));' for f in fields_p]
    lines += ['return 0;}']
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", f"-I{ROOT / 'include'}", str(src),
                    "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split()
    assert [int(out[0]), int(out[1])] == [C.sizeof(api.ReduceDesc), C.sizeof(api.Plan)]
    offs = [int(x) for x in out[2:]]
    want = [getattr(api.ReduceDesc, f).offset for f in fields_d] + \
           [getattr(api.Plan, f).offset for f in fields_p]
    assert offs == want
    lib = api.load()
    for dt, size in api.DTYPE_SIZE.items():
        assert lib.rmi_dtype_size(dt) == size
    assert lib.rmi_dtype_size(99) == 0


def test_status_strings():
    lib = api.load()
    seen = {lib.rmi_status_string(i).decode() for i in range(10)}
    assert len(seen) == 10 and "ok" in seen
    assert lib.rmi_status_string(1234).decode() == "unknown status"


BENCH_SHAPES = [
    # in, out, rows, cols, kwargs, expected plan, expected passes
    (api.F32, api.F32, 10000, 256, {}, api.PLAN_ROW_WAVE, 1),
    (api.F32, api.F32, 1000000, 128, dict(main_op=api.MAIN_SQ, final_op=api.FIN_SQRT),
     api.PLAN_ROW_WAVE, 1),
    (api.F32, api.F32, 10000000, 64, dict(apply=api.ALONG_COLUMNS), api.PLAN_COL_TILE, 2),
    (api.F32, api.KVP_I32_F32, 65536, 32000,
     dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX), api.PLAN_ROW_BLOCK, 1),
    (api.I8, api.I64, 4096, 16384, {}, api.PLAN_ROW_BLOCK, 1),
    (api.I8, api.I64, 16777216, 8, {}, api.PLAN_ROW_LANES, 1),
    (api.I8, api.I64, 16777216, 4, {}, api.PLAN_ROW_WAVE, 1),           # four rows per vector: through LDS
    (api.BF16, api.F32, 8, 4194304, {}, api.PLAN_ROW_SPLIT, 2),
]


@pytest.mark.parametrize("in_dt,out_dt,rows,cols,kw,plan,passes", BENCH_SHAPES)
def test_plans_of_benchmark_shapes(in_dt, out_dt, rows, cols, kw, plan, passes):
    d = api.make_desc(in_dt, out_dt, rows, cols, **kw)
    p = api.plan_query(d)
    assert p.kind == plan and p.passes == passes
    assert p.vec_bytes == 16
    n_out = cols if kw.get("apply") == api.ALONG_COLUMNS else rows
    assert p.n_outputs == n_out and p.reduce_len == rows * cols // n_out
    ws = api.load().rmi_reduce_workspace_bytes(C.byref(d))
    assert (ws > 0) == (passes == 2)
    assert ws >= p.workspace_bytes
    assert p.grid_blocks >= 1


def test_plan_hints_and_fallbacks():
    # a forced split on a short row degrades to one block per row
    d = api.make_desc(api.F32, api.F32, 10, 512, plan_hint=api.PLAN_ROW_SPLIT)
    p = api.plan_query(d)
    assert p.kind == api.PLAN_ROW_BLOCK and p.passes == 1 and p.workspace_bytes == 0
    d = api.make_desc(api.F32, api.F32, 4, 1 << 20, plan_hint=api.PLAN_ROW_SPLIT)
    p = api.plan_query(d)
    assert p.kind == api.PLAN_ROW_SPLIT and p.blocks_per_out >= 2
    assert p.workspace_bytes == api.WORKSPACE_TICKET_BYTES + 4 * p.blocks_per_out * 8
    # rows of 7 floats (28 B) are one 16-byte vector plus three tail elements;
    # rows of 3 floats (12 B) go through LDS as whole vectors, and are read element by element
    # when the lane-group plan is asked for
    p = api.plan_query(api.make_desc(api.F32, api.F32, 1000, 7))
    assert p.vec_bytes == 16 and p.kind == api.PLAN_ROW_WAVE
    p = api.plan_query(api.make_desc(api.F32, api.F32, 1000, 3))
    assert p.vec_bytes == 16 and p.kind == api.PLAN_ROW_WAVE and p.lanes_per_row == 1
    p = api.plan_query(api.make_desc(api.F32, api.F32, 1000, 3, plan_hint=api.PLAN_ROW_WAVE))
    assert p.vec_bytes == 4 and p.kind == api.PLAN_ROW_WAVE
    # f64 sums carry a 16-byte (sum, compensation) accumulator through the partials
    d = api.make_desc(api.F64, api.F64, 4, 1 << 20, plan_hint=api.PLAN_ROW_SPLIT)
    p = api.plan_query(d)
    assert p.workspace_bytes == api.WORKSPACE_TICKET_BYTES + 4 * p.blocks_per_out * 16
    # with zeroed ticket words in the workspace the last workgroup of a row folds: one launch
    d.flags = api.FLAG_WORKSPACE_ZEROED
    p1 = api.plan_query(d)
    assert (p1.kind, p1.passes, p1.workspace_bytes) == (api.PLAN_ROW_SPLIT, 1, p.workspace_bytes)
    # column-major along rows is a strided fold
    p = api.plan_query(api.make_desc(api.F32, api.F32, 64, 100000, layout=api.COL_MAJOR))
    assert p.kind == api.PLAN_COL_TILE and p.n_outputs == 64


@pytest.mark.parametrize("kw,status", [
    (dict(in_dtype=77), api.ERR_BAD_ENUM),
    (dict(layout=5), api.ERR_BAD_ENUM),
    (dict(reduce_op=9), api.ERR_BAD_ENUM),
    (dict(n_rows=-3), api.ERR_BAD_SHAPE),
    (dict(out_dtype=api.I64), api.ERR_UNSUPPORTED),             # float in, int out
    (dict(out_dtype=api.KVP_I32_F32), api.ERR_UNSUPPORTED),     # KVP out needs an arg-reduce
    (dict(reduce_op=api.RED_ARGMAX), api.ERR_UNSUPPORTED),      # arg-reduce needs MAIN_KVP
    (dict(reduce_op=api.RED_ARGMAX, main_op=api.MAIN_KVP, out_dtype=api.KVP_I32_F64),
     api.ERR_UNSUPPORTED),                                      # value type mismatch
    (dict(final_op=api.FIN_STDDEV_FROM_SUMSQ), api.ERR_NULL),   # needs final_aux
    (dict(in_dtype=api.KVP_I32_F32), api.ERR_UNSUPPORTED),
    (dict(flags=2), api.ERR_BAD_ENUM),
])
def test_descriptor_validation(kw, status):
    d = api.make_desc(api.F32, api.F32, 100, 100)
    for k, v in kw.items():
        setattr(d, k, v)
    p = api.Plan()
    assert api.load().rmi_plan_query(C.byref(d), C.byref(p)) == status


def test_null_and_workspace_errors_without_a_launch():
    lib = api.load()
    p = api.Plan()
    assert lib.rmi_plan_query(None, C.byref(p)) == api.ERR_NULL
    d = api.make_desc(api.F32, api.F32, 100, 100)
    assert lib.rmi_plan_query(C.byref(d), None) == api.ERR_NULL
    assert lib.rmi_reduce(None, None, None, None, 0, None) == api.ERR_NULL
    # the checks below return before anything is launched
    assert lib.rmi_reduce(C.byref(d), 0x1000, None, None, 0, None) == api.ERR_NULL
    assert lib.rmi_reduce(C.byref(d), None, 0x1000, None, 0, None) == api.ERR_NULL
    assert lib.rmi_reduce(C.byref(d), 0x1002, 0x1000, None, 0, None) == api.ERR_ALIGNMENT
    assert lib.rmi_reduce(C.byref(d), 0x1000, 0x1002, None, 0, None) == api.ERR_ALIGNMENT
    d = api.make_desc(api.BF16, api.F32, 8, 4194304)
    assert lib.rmi_reduce(C.byref(d), 0x1000, 0x2000, None, 0, None) == api.ERR_WORKSPACE
    assert lib.rmi_reduce(C.byref(d), 0x1000, 0x2000, 0x3000, 16, None) == api.ERR_WORKSPACE
    assert lib.rmi_map_reduce(C.byref(d), -1, None, None, None, 0, None) == api.ERR_BAD_SHAPE
    dn = api.make_desc(api.I8, api.I8, 10, 10)
    assert lib.rmi_row_normalize(C.byref(dn), 0x1000, 0x2000, 1e-8, None) == api.ERR_UNSUPPORTED
    dn = api.make_desc(api.F32, api.F32, 10, 10, final_op=api.FIN_SQ)
    assert lib.rmi_row_normalize(C.byref(dn), 0x1000, 0x2000, 1e-8, None) == api.ERR_UNSUPPORTED
    dn = api.make_desc(api.F32, api.F32, 10, 10)
    assert lib.rmi_row_normalize(C.byref(dn), None, 0x2000, 1e-8, None) == api.ERR_NULL
    assert lib.rmi_row_normalize(C.byref(dn), 0x1002, 0x2000, 1e-8, None) == api.ERR_ALIGNMENT
    dn = api.make_desc(api.F32, api.F32, 0, 10)
    assert lib.rmi_row_normalize(C.byref(dn), None, None, 1e-8, None) == api.OK
    # zero outputs: success, nothing to do
    d = api.make_desc(api.F32, api.F32, 0, 100)
    assert lib.rmi_reduce(C.byref(d), None, None, None, 0, None) == api.OK


def test_lane_groups_follow_the_row_length():
    """Rows whose lane-load count is far from a power of two get one lane per lane-load
    (5 lane-loads, and 6 or 9..17 with tail elements); the others keep power-of-two groups."""
    lanes = lambda cols, dt=api.F32, out=api.F32, hint=api.PLAN_AUTO: api.plan_query(
        api.make_desc(dt, out, 1000000, cols, plan_hint=hint)).lanes_per_row
    assert lanes(20) == 5 and lanes(17) == 5            # 5 lane-loads, without and with a tail
    assert lanes(33) == 9 and lanes(45) == 12 and lanes(62) == 16
    # 17, 18 and 33 lane-loads with a tail: the row's own count (slots dealt over whole rows)
    assert lanes(66) == 17 and lanes(70) == 18 and lanes(129) == 33 and lanes(68) == 8
    assert lanes(83) == 21 and lanes(125) == 32 and lanes(90) == 8   # 23 lane-loads: 46 lanes, no
    assert lanes(21) == 6                               # 5 whole vectors + one element
    assert lanes(24) == 8 and lanes(28) == 8            # 6 and 7 whole lane-loads stay on 8 lanes
    assert lanes(36) == 4                               # 9 whole vectors: 4 lanes x 3 loads
    assert lanes(128) == 8 and lanes(256) == 16
    # 16-bit and 8-byte rows of up to 512 bytes that are no whole vectors go through LDS, a
    # thread per row; the lane groups serve them when the plan is asked for (or the input
    # starts off a 16-byte boundary)
    W = api.PLAN_ROW_WAVE
    assert lanes(100, api.BF16) == 1 and lanes(17, api.F64, api.F64) == 1 and lanes(9) == 1
    assert lanes(100, api.BF16, hint=W) == 13           # 12 whole + 4 elements
    # 16-byte accumulators (f64 sums) keep it up to 12 lane-loads
    assert lanes(17, api.F64, api.F64, W) == 9 and lanes(63, api.F64, api.F64, W) == 8
    # (with a tail they take their own count again from 5 to 18 lane-loads, whole rows dealt over
    # the workgroup's load slots, under the automatic plan only: inputs off a 16-byte boundary)
    assert lanes(25, api.F64, api.F64, W) == 8
    # arg-reductions follow the same rule
    d = api.make_desc(api.F32, api.KVP_I32_F32, 1000, 33, main_op=api.MAIN_KVP,
                      reduce_op=api.RED_ARGMAX)
    assert api.plan_query(d).lanes_per_row == 9


def test_column_plans_of_rows_that_are_not_whole_vectors():
    """Rows shorter than 16 bytes are folded in groups of rows that make whole vectors (more
    partials per output, a second pass), unless the reduction needs the row index or the
    matrix is short; the workspace query covers the plan an unaligned input falls back to."""
    lib = api.load()
    d = api.make_desc(api.F32, api.F32, 4_000_000, 3, apply=api.ALONG_COLUMNS)
    p = api.plan_query(d)
    assert p.kind == api.PLAN_COL_TILE and p.passes == 2 and p.vec_bytes == 16
    assert p.blocks_per_out % 4 == 0                    # 4 rows of 12 bytes = 3 vectors
    assert lib.rmi_reduce_workspace_bytes(C.byref(d)) >= p.workspace_bytes
    d = api.make_desc(api.I8, api.I64, 4_000_000, 5, apply=api.ALONG_COLUMNS)
    assert api.plan_query(d).blocks_per_out % 16 == 0   # 16 rows of 5 bytes = 5 vectors
    d = api.make_desc(api.F32, api.KVP_I32_F32, 4_000_000, 3, apply=api.ALONG_COLUMNS,
                      main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMIN)
    assert api.plan_query(d).vec_bytes == 4             # element by element
    d = api.make_desc(api.F32, api.F32, 500, 3, apply=api.ALONG_COLUMNS)
    assert api.plan_query(d).vec_bytes == 4             # too few rows to group
    # wider rows are never grouped: one partial per workgroup row
    d = api.make_desc(api.F32, api.F32, 1_000_000, 129, apply=api.ALONG_COLUMNS)
    p = api.plan_query(d)
    assert p.kind == api.PLAN_COL_TILE and p.vec_bytes == 16 and p.blocks_per_out <= 4096
    assert p.grid_blocks == p.blocks_per_out            # 33 lane-loads: one workgroup column


def test_column_plans_of_wide_rows():
    """Floating sums, max and min down rows of more than 128 lane-loads: whole adjacent rows
    per workgroup (one workgroup per CU of the 256 a build host is planned for, one set of
    partials each, a second pass), rows beyond 1280 lane-loads in the fewest equal pieces;
    byte sums likewise where their rows fill three quarters of the 1024 slots, arg-reductions
    too; short matrices and whole multiples of 64 lane-loads in several pieces keep the other
    layout;
    the library's own descriptor flag is refused."""
    lib = api.load()
    q = lambda rows, cols, in_dt=api.F32, out_dt=api.F32, **kw: api.plan_query(
        api.make_desc(in_dt, out_dt, rows, cols, apply=api.ALONG_COLUMNS, **kw))
    p = q(32768, 4097)
    assert (p.kind, p.passes, p.grid_blocks, p.blocks_per_out) == (api.PLAN_COL_TILE, 2, 256, 256)
    assert p.workspace_bytes == api.WORKSPACE_TICKET_BYTES + 4097 * 256 * 8
    p = q(16384, 11000)                                  # 2750 lane-loads: three pieces of 917
    assert (p.grid_blocks, p.blocks_per_out) == (3 * 85, 85)
    p = q(16384, 4097, api.F64, api.F64)                 # compensated sums: 16-byte partials
    assert p.grid_blocks == 2 * 128 and p.workspace_bytes == api.WORKSPACE_TICKET_BYTES + 4097 * 128 * 16
    assert q(8191, 4097).grid_blocks != 256              # fewer than sixteen steps per workgroup
    assert q(4096, 32768).grid_blocks > 256              # 8192 whole lane-loads: pieces of 64 lanes
    kvp = dict(main_op=api.MAIN_KVP, reduce_op=api.RED_ARGMAX)
    p = q(32768, 4097, api.F32, api.KVP_I32_F32, **kvp)
    assert (p.passes, p.grid_blocks, p.blocks_per_out) == (2, 256, 256)
    p = q(131072, 4100, api.I8, api.I64)                 # 257 lane-loads, three rows per bundle
    assert (p.kind, p.passes, p.grid_blocks, p.blocks_per_out) == (api.PLAN_COL_TILE, 2, 256, 256)
    assert q(131072, 4100, api.I8, api.F32).grid_blocks == 256
    assert q(65536, 8200, api.I8, api.I64).grid_blocks > 256    # 513 lane-loads: half of the slots
    assert q(131072, 4096, api.I8, api.I64).grid_blocks > 256   # whole multiples of 64 lane-loads
    assert q(131072, 4100, api.I8, api.I64, reduce_op=api.RED_MAX, init_i=-128).grid_blocks > 256
    d = api.make_desc(api.F32, api.F32, 32768, 4097, apply=api.ALONG_COLUMNS, flags=1 << 30)
    plan = api.Plan()
    assert lib.rmi_plan_query(C.byref(d), C.byref(plan)) == api.ERR_BAD_ENUM
    assert lib.rmi_reduce_workspace_bytes(C.byref(d)) == 0
