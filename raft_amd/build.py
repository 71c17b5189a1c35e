"""Build recipe for the native parts: the gfx950 reduction library
(raft_amd/lib/libraft_amd.so, C ABI in include/rmi_reduce.h), the CPU oracle
(oracle/liboracle.so) and the C++ API test programs (tests/cpp/bin/*).

Everything is built in-tree with explicit compiler command lines; hipcc
cross-compiles for gfx950 without a GPU present.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
CSRC = ROOT / "raft_amd" / "csrc"
LIBDIR = ROOT / "raft_amd" / "lib"
OBJDIR = LIBDIR / "obj"
LIB = LIBDIR / "libraft_amd.so"
CXX_API_INCLUDE = ROOT / "raft_amd" / "include"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
]


def _run(cmd: list[str], quiet_pattern: str | None = None) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = proc.stdout
    if quiet_pattern:
        out = "\n".join(l for l in out.splitlines() if quiet_pattern not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(map(str, cmd))}\n{out}")
    if out.strip():
        sys.stderr.write(out + "\n")


def _jobs() -> int:
    return max(1, min(8, os.cpu_count() or 1, int(os.environ.get("MAX_JOBS", "8"))))


def build_library(force: bool = True) -> Path:
    """Compile every .hip translation unit for gfx950 and link the shared library."""
    OBJDIR.mkdir(parents=True, exist_ok=True)
    sources = sorted(CSRC.glob("*.hip"))
    headers = list(CSRC.glob("*.hpp")) + [ROOT / "include" / "rmi_reduce.h"]
    newest_header = max(h.stat().st_mtime for h in headers)

    def compile_one(src: Path) -> Path:
        obj = OBJDIR / (src.stem + ".o")
        if (not force and obj.exists()
                and obj.stat().st_mtime > max(src.stat().st_mtime, newest_header)):
            return obj
        _run([HIPCC, *HIP_FLAGS, "-c", str(src), "-o", str(obj)],
             quiet_pattern="packed-fp32-ops")
        return obj

    with ThreadPoolExecutor(max_workers=_jobs()) as pool:
        objs = list(pool.map(compile_one, sources))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)],
         quiet_pattern="packed-fp32-ops")
    return LIB


def build_oracle() -> Path:
    """Compile the CPU oracle (test infrastructure, never part of the product path)."""
    _run(["make", "-s", "-C", str(ROOT / "oracle")])
    return ROOT / "oracle" / "liboracle.so"


def build_cpp_tests() -> list[Path]:
    """Compile the host-side C++ API test programs with g++ against the headers."""
    tdir = ROOT / "tests" / "cpp"
    if not (tdir / "Makefile").exists():
        return []
    _run(["make", "-s", "-C", str(tdir)])
    return sorted((tdir / "bin").glob("*"))


def build_bench() -> list[Path]:
    """Compile the benchmark program over the reference's shape grids (hipcc)."""
    bdir = ROOT / "raft_amd" / "bench"
    _run(["make", "-s", "-C", str(bdir)])
    return sorted((bdir / "bin").glob("*"))


def build_all(force: bool = True) -> None:
    build_library(force=force)
    build_oracle()
    build_cpp_tests()
    build_bench()


if __name__ == "__main__":
    build_all(force="--incremental" not in sys.argv)
    print(f"built {LIB}")
