// raft::resources as far as the reduction path needs it: the stream every
// call is ordered on, and a device workspace that multi-pass plans reuse
// between calls.  The reference's registry of lazily built resources
// (core/resources.hpp:47-143) is reduced to these two.
//
// Like the reference's handle, one raft::resources must not be used from two
// host threads at once; calls made through it are ordered on its stream, which
// is also what makes sharing its workspace between consecutive calls safe.
// Copies share the workspace (the reference's copies share their resources the
// same way) and carry a stream of their own.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <memory>

#include <raft/core/error.hpp>

#include "rmi_reduce.h"

namespace raft {

class resources {
 public:
  // Default stream: the per-thread default stream, as in the reference
  // (core/resource/cuda_stream.hpp:23).
  resources() : ws_(std::make_shared<workspace_state>()) {}
  explicit resources(hipStream_t stream) : stream_(stream), ws_(std::make_shared<workspace_state>()) {}
  resources(const resources&)            = default;
  resources& operator=(const resources&) = default;
  resources(resources&&)                 = default;
  resources& operator=(resources&&)      = default;
  virtual ~resources()                   = default;

  hipStream_t get_stream() const { return stream_; }
  void set_stream(hipStream_t s) { stream_ = s; }
  void sync_stream() const { RAFT_HIP_TRY(hipStreamSynchronize(stream_)); }

  // Device scratch of at least `bytes` bytes, 256-byte aligned, valid until the next call
  // that asks for more.  Work that used it earlier is ordered before the caller's: on the
  // same stream by the stream itself; when the handle's stream has changed since (or
  // the buffer has to grow) by waiting for the stream that used it last.  Its first
  // RMI_WORKSPACE_TICKET_BYTES bytes are zeroed when it is allocated and only the library
  // writes there, which is what RMI_FLAG_WORKSPACE_ZEROED asks of a workspace.
  void* workspace(size_t bytes) const
  {
    workspace_state& w = *ws_;
    if (w.used && (w.last != stream_ || bytes > w.bytes)) {
      RAFT_HIP_TRY(hipStreamSynchronize(w.last));
      w.used = false;
    }
    if (bytes > w.bytes) {
      if (w.ptr != nullptr) {
        RAFT_HIP_TRY(hipFree(w.ptr));
        w.ptr   = nullptr;
        w.bytes = 0;
      }
      const size_t want = bytes < (size_t(1) << 20) ? (size_t(1) << 20) : bytes;
      RAFT_HIP_TRY(hipMalloc(&w.ptr, want));
      w.bytes = want;
      RAFT_HIP_TRY(hipMemset(w.ptr, 0, RMI_WORKSPACE_TICKET_BYTES));
    }
    w.last = stream_;
    w.used = true;
    return w.ptr;
  }

  // 256 bytes of device memory for scalars that one call of a primitive hands to its next
  // kernel (the weight sum of weighted_mean); separate from the workspace, allocated at the
  // first use, ordered like the workspace.
  void* scalars() const
  {
    workspace_state& w = *ws_;
    if (w.scalars_used && w.scalars_last != stream_) RAFT_HIP_TRY(hipStreamSynchronize(w.scalars_last));
    if (w.scalars == nullptr) RAFT_HIP_TRY(hipMalloc(&w.scalars, 256));
    w.scalars_last = stream_;
    w.scalars_used = true;
    return w.scalars;
  }

 private:
  struct workspace_state {
    void* ptr        = nullptr;
    size_t bytes     = 0;
    hipStream_t last = nullptr;  // the stream of the last call that used the buffer
    bool used        = false;    // work that uses the buffer may still be queued on `last`
    void* scalars            = nullptr;
    hipStream_t scalars_last = nullptr;
    bool scalars_used        = false;
    workspace_state()                                  = default;
    workspace_state(const workspace_state&)            = delete;
    workspace_state& operator=(const workspace_state&) = delete;
    ~workspace_state()
    {
      if (ptr != nullptr) {
        if (used) (void)hipStreamSynchronize(last);
        (void)hipFree(ptr);
      }
      if (scalars != nullptr) {
        if (scalars_used) (void)hipStreamSynchronize(scalars_last);
        (void)hipFree(scalars);
      }
    }
  };

  hipStream_t stream_ = hipStreamPerThread;
  std::shared_ptr<workspace_state> ws_;
};

}  // namespace raft
