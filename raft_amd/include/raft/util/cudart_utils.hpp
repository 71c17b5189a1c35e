// Stream-ordered copies between host and device (util/cudart_utils.hpp:137-193
// in the reference), over the HIP runtime.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstddef>

#include <raft/core/error.hpp>

namespace raft {

template <typename T>
void copy(T* dst, const T* src, size_t len, hipStream_t stream)
{
  if (len == 0) return;
  RAFT_HIP_TRY(hipMemcpyAsync(dst, src, len * sizeof(T), hipMemcpyDefault, stream));
}
template <typename T>
void update_device(T* d_ptr, const T* h_ptr, size_t len, hipStream_t stream)
{
  copy(d_ptr, h_ptr, len, stream);
}
template <typename T>
void update_host(T* h_ptr, const T* d_ptr, size_t len, hipStream_t stream)
{
  copy(h_ptr, d_ptr, len, stream);
}

template <typename IntT>
constexpr IntT ceildiv(IntT a, IntT b)
{
  return (a + b - 1) / b;
}

}  // namespace raft
