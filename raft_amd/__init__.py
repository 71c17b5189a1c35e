"""raft_amd — MI355X-native dense reductions behind RAFT's reduce()/norm()/mean() API.

The product is the shared library raft_amd/lib/libraft_amd.so (hand-written
gfx950 HIP kernels, C ABI in include/rmi_reduce.h) and the C++ headers under
raft_amd/include that keep the reference's template API on top of it.  The
Python in this package is plumbing for tests and benchmarks: a ctypes view of
the C ABI (`_capi`) and helpers that pass torch device tensors through it
(`device`).
"""
__all__ = ["_capi", "build", "device"]
