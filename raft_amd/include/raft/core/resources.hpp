// raft::resources as far as the reduction path needs it: the stream every
// call is ordered on, and a device workspace that multi-pass plans reuse
// between calls.  The reference's registry of lazily built resources
// (core/resources.hpp:47-143) is reduced to these two.
//
// Like the reference's handle, one raft::resources must not be used from two
// host threads at once; calls made through it are ordered on its stream, which
// is also what makes sharing its workspace between consecutive calls safe.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstddef>

#include <raft/core/error.hpp>

namespace raft {

class resources {
 public:
  // Default stream: the per-thread default stream, as in the reference
  // (core/resource/cuda_stream.hpp:23).
  resources() = default;
  explicit resources(hipStream_t stream) : stream_(stream) {}
  resources(const resources&)            = delete;
  resources& operator=(const resources&) = delete;
  virtual ~resources()
  {
    if (workspace_ != nullptr) {
      (void)hipStreamSynchronize(stream_);
      (void)hipFree(workspace_);
    }
  }

  hipStream_t get_stream() const { return stream_; }
  void set_stream(hipStream_t s) { stream_ = s; }
  void sync_stream() const { RAFT_HIP_TRY(hipStreamSynchronize(stream_)); }

  // Device scratch of at least `bytes` bytes, 256-byte aligned, valid until the
  // next call that asks for more.  Growing waits for the stream first.
  void* workspace(size_t bytes) const
  {
    if (bytes <= workspace_bytes_) return workspace_;
    if (workspace_ != nullptr) {
      RAFT_HIP_TRY(hipStreamSynchronize(stream_));
      RAFT_HIP_TRY(hipFree(workspace_));
      workspace_       = nullptr;
      workspace_bytes_ = 0;
    }
    size_t want = bytes < (size_t(1) << 20) ? (size_t(1) << 20) : bytes;
    RAFT_HIP_TRY(hipMalloc(&workspace_, want));
    workspace_bytes_ = want;
    return workspace_;
  }

 private:
  hipStream_t stream_ = hipStreamPerThread;
  mutable void* workspace_        = nullptr;
  mutable size_t workspace_bytes_ = 0;
};

}  // namespace raft
