#pragma once
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/core/resources.hpp>

namespace raft {
// The convenience handle of the reference (core/device_resources.hpp), as far as
// the reduction path uses it.
class device_resources : public resources {
 public:
  using resources::resources;
};
}  // namespace raft
