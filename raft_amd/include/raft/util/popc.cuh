// raft::popc (util/popc.cuh:14-33 in the reference): counts the set bits among the first
// max_len bits of `values` into `counter`.  Compile with hipcc.
#pragma once

#include <raft/util/detail/popc.cuh>

namespace raft {

template <typename value_t, typename index_t>
void popc(const raft::resources& res,
          device_vector_view<const value_t, index_t> values,
          raft::host_scalar_view<const index_t, index_t> max_len,
          raft::device_scalar_view<index_t> counter)
{
  detail::popc(res, values, max_len, counter);
}

}  // namespace raft
