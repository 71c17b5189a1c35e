// Stream accessors of a raft::resources (core/resource/cuda_stream.hpp:62-107 in
// the reference).  The names are kept so that callers compile unchanged; the
// stream type is hipStream_t.
#pragma once

#include <raft/core/resources.hpp>

namespace raft::resource {

inline hipStream_t get_cuda_stream(resources const& res) { return res.get_stream(); }
inline void set_cuda_stream(resources& res, hipStream_t stream) { res.set_stream(stream); }
inline void sync_stream(resources const& res, hipStream_t stream)
{
  (void)res;
  RAFT_HIP_TRY(hipStreamSynchronize(stream));
}
inline void sync_stream(resources const& res) { res.sync_stream(); }

}  // namespace raft::resource
