// Stream-ordered scratch memory for callers that pass a bare stream and no handle:
// a memory pool owned by this library, one per device, whose freed blocks stay
// cached for the next call.  It plays the role the reference's rmm pool plays for
// its per-call rmm::device_uvector workspaces
// (linalg/detail/coalesced_reduction-inl.cuh:560).
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <map>
#include <mutex>

#include <raft/core/error.hpp>

namespace raft::detail::rmi {

inline hipMemPool_t scratch_pool()
{
  static std::mutex guard;
  static std::map<int, hipMemPool_t> by_device;
  int dev = 0;
  RAFT_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(guard);
  auto it = by_device.find(dev);
  if (it != by_device.end()) return it->second;
  hipMemPoolProps props{};
  props.allocType     = hipMemAllocationTypePinned;
  props.handleTypes   = hipMemHandleTypeNone;
  props.location.type = hipMemLocationTypeDevice;
  props.location.id   = dev;
  hipMemPool_t pool   = nullptr;
  RAFT_HIP_TRY(hipMemPoolCreate(&pool, &props));
  // keep freed blocks instead of returning them to the driver at every synchronisation
  std::uint64_t keep = UINT64_MAX;
  RAFT_HIP_TRY(hipMemPoolSetAttribute(pool, hipMemPoolAttrReleaseThreshold, &keep));
  by_device.emplace(dev, pool);
  return pool;
}

inline void* scratch_alloc(std::size_t bytes, hipStream_t stream)
{
  void* p = nullptr;
  RAFT_HIP_TRY(hipMallocFromPoolAsync(&p, bytes, scratch_pool(), stream));
  return p;
}

inline void scratch_free(void* p, hipStream_t stream)
{
  if (p != nullptr) (void)hipFreeAsync(p, stream);
}

}  // namespace raft::detail::rmi
