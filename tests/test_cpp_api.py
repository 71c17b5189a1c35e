"""Runs the C++ API test programs (tests/cpp/*.cpp, built by raft_amd.build).

test_raft_host needs no GPU: functor vocabulary, views, precondition errors, plan
selector.  test_raft_api restates the reference's reduction-path tests against the
kept raft:: names and runs on the GPU.  test_raft_generic is compiled by hipcc and
covers functors outside the library's vocabulary."""
import subprocess
from pathlib import Path

import pytest

BIN = Path(__file__).resolve().parent / "cpp" / "bin"


def _run(name, timeout):
    exe = BIN / name
    if not exe.exists():
        from raft_amd import build
        build.build_cpp_tests()
    proc = subprocess.run([str(exe)], capture_output=True, text=True, timeout=timeout)
    tail = "\n".join(proc.stdout.splitlines()[-40:])
    assert proc.returncode == 0, f"{name} failed (rc={proc.returncode}):\n{tail}\n{proc.stderr[-2000:]}"
    return proc.stdout


def test_cpp_host_layer():
    out = _run("test_raft_host", 60)
    assert "0 failed" in out


def test_plan_selector_properties():
    """400000 random and extreme descriptors through the plan selector under ASan / UBSan
    (tests/cpp/test_plan_fuzz.cpp): the invariants kernels and host checks rely on."""
    out = _run("test_plan_fuzz", 120)
    assert "0 failed" in out


@pytest.mark.gpu
def test_cpp_api_on_gpu(gpu):
    out = _run("test_raft_api", 600)
    assert "0 failed" in out


@pytest.mark.gpu
def test_cpp_generic_functors_on_gpu(gpu):
    """Device lambdas, caller-defined functors and KeyValuePair<int, short>, instantiated in
    a hipcc translation unit by the header fallback (tests/cpp/test_raft_generic.hip)."""
    out = _run("test_raft_generic", 600)
    assert "0 failed" in out


@pytest.mark.gpu
def test_cpp_map_family_on_gpu(gpu):
    """raft::linalg::map / map_offset / unaryOp / writeOnlyUnaryOp / binaryOp
    (tests/cpp/test_raft_map.hip, compiled by hipcc)."""
    out = _run("test_raft_map", 600)
    assert "0 failed" in out


@pytest.mark.gpu
def test_bench_program_runs_on_gpu(gpu):
    """The benchmark program over the reference's shape grids starts, runs one small grid
    and prints one line per case (raft_amd/bench/prims_bench.hip)."""
    exe = BIN.parent.parent.parent / "raft_amd" / "bench" / "bin" / "prims_bench"
    if not exe.exists():
        from raft_amd import build
        build.build_bench()
    proc = subprocess.run([str(exe), "--filter", "rowNorm<float,int>", "--min-iters", "2"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    lines = [l for l in proc.stdout.splitlines() if l.startswith("rowNorm<float,int>")]
    assert len(lines) == 35 and all("GB/s" in l for l in lines)
