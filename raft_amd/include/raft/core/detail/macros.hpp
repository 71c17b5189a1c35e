// Function-decoration macros used by the headers of the reduction path.
// Host and device code of this build are separate translation units (the
// kernels live in libraft_amd.so), so the decorations only matter when a
// header is also read by hipcc.
#pragma once

#if defined(__HIPCC__)
#define RAFT_HOST_DEVICE __host__ __device__
#else
#define RAFT_HOST_DEVICE
#endif
#define RAFT_INLINE_FUNCTION inline RAFT_HOST_DEVICE
#ifndef HDI
#define HDI RAFT_INLINE_FUNCTION
#endif
#define RAFT_EXPORT
