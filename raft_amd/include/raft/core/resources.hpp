// raft::resources as far as the reduction path needs it: the stream every
// call is ordered on, and a device workspace that multi-pass plans reuse
// between calls.  The reference's registry of lazily built resources
// (core/resources.hpp:47-143) is reduced to these two.
//
// After its first use a handle neither allocates nor makes the host wait: the workspace
// comes from a stream-ordered pool and is kept, a change of the handle's stream is ordered
// with an event (the new stream waits on the device for the work the old one still holds),
// and the ticket words are cleared by a kernel.  Calls through a warmed-up handle can
// therefore be recorded into a HIP graph, as the reference's stream-ordered contract allows
// (core/resource/cuda_stream.hpp:62-107, linalg/detail/coalesced_reduction-inl.cuh:560).
//
// Copies share the workspace (the reference's copies share their resources the same way)
// and carry a stream of their own; the bookkeeping is guarded, so copies may be used from
// several host threads, their calls then taking turns on the device.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <memory>
#include <mutex>

#include <raft/core/error.hpp>
#include <raft/linalg/detail/rmi_scratch.hpp>

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
  // same stream by the stream itself, after a change of stream by an event that the new
  // stream waits for (no host wait).  Its first RMI_WORKSPACE_TICKET_BYTES bytes are zeroed
  // by a kernel when it is allocated and only the library writes there, which is what
  // RMI_FLAG_WORKSPACE_ZEROED asks of a workspace.  Growing allocates from the pool on the
  // handle's stream and hands the old buffer back on it: no device-wide synchronisation, but
  // an allocation, so the sizes a captured sequence needs have to be reached before capture.
  void* workspace(size_t bytes) const
  {
    workspace_state& w = *ws_;
    std::lock_guard<std::mutex> lock(w.guard);
    w.follow(w.last, w.used, stream_);
    if (bytes > w.bytes) {
      const size_t want = bytes < kFirstBytes ? kFirstBytes : bytes;
      void* fresh       = detail::rmi::scratch_alloc(want, stream_);
      const int rc      = rmi_workspace_reset(fresh, want, stream_);
      if (rc != RMI_OK) {
        detail::rmi::scratch_free(fresh, stream_);
        RAFT_FAIL("rmi_workspace_reset: %s", rmi_status_string(rc));
      }
      // everything that used the old buffer is ordered before this point of stream_
      detail::rmi::scratch_free(w.ptr, stream_);
      w.ptr   = fresh;
      w.bytes = want;
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
    std::lock_guard<std::mutex> lock(w.guard);
    w.follow(w.scalars_last, w.scalars_used, stream_);
    if (w.scalars == nullptr) w.scalars = detail::rmi::scratch_alloc(256, stream_);
    w.scalars_last = stream_;
    w.scalars_used = true;
    return w.scalars;
  }

 private:
  // first allocation: holds the partials of every plan of the reduction family at the
  // shapes of the benchmark configs (the largest, meanvar of 64 columns, needs 1.1 MB)
  static constexpr size_t kFirstBytes = size_t(8) << 20;

  struct workspace_state {
    std::mutex guard;
    void* ptr        = nullptr;
    size_t bytes     = 0;
    hipStream_t last = nullptr;  // the stream of the last call that used the buffer
    bool used        = false;    // work that uses the buffer may still be queued on `last`
    void* scalars            = nullptr;
    hipStream_t scalars_last = nullptr;
    bool scalars_used        = false;
    hipEvent_t order         = nullptr;  // made at the first change of stream
    workspace_state()                                  = default;
    workspace_state(const workspace_state&)            = delete;
    workspace_state& operator=(const workspace_state&) = delete;

    // Orders `next` after the work queued on `last`, on the device.
    void follow(hipStream_t last_stream, bool in_use, hipStream_t next)
    {
      if (!in_use || last_stream == next) return;
      if (order == nullptr) RAFT_HIP_TRY(hipEventCreateWithFlags(&order, hipEventDisableTiming));
      RAFT_HIP_TRY(hipEventRecord(order, last_stream));
      RAFT_HIP_TRY(hipStreamWaitEvent(next, order, 0));
    }

    ~workspace_state()
    {
      // hand the buffers back behind the work that may still use them
      if (ptr != nullptr) (void)hipFreeAsync(ptr, last);
      if (scalars != nullptr) (void)hipFreeAsync(scalars, scalars_last);
      if (order != nullptr) (void)hipEventDestroy(order);
    }
  };

  hipStream_t stream_ = hipStreamPerThread;
  std::shared_ptr<workspace_state> ws_;
};

}  // namespace raft
