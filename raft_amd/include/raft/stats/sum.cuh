// Column sums (stats/sum.cuh:35-74, stats/detail/sum.cuh:17-21 in the reference).
#pragma once

#include <raft/core/device_mdspan.hpp>
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/linalg/detail/rmi_bridge.hpp>

namespace raft::stats {

template <bool rowMajor, typename Type, typename IdxType = int>
void sum(Type* output, const Type* input, IdxType D, IdxType N, hipStream_t stream)
{
  raft::detail::rmi::reduce(nullptr, stream, output, input, (std::int64_t)N, (std::int64_t)D,
                            rowMajor, false, raft::detail::rmi::zero<Type>(), false, raft::identity_op(), raft::add_op(),
                            raft::identity_op());
}

template <typename value_t, typename idx_t, typename layout_t>
void sum(raft::resources const& handle,
         raft::device_matrix_view<const value_t, idx_t, layout_t> input,
         raft::device_vector_view<value_t, idx_t> output)
{
  constexpr bool is_row_major = std::is_same_v<layout_t, raft::row_major>;
  static_assert(is_row_major || std::is_same_v<layout_t, raft::col_major>,
                "sum: Layout must be either "
                "raft::row_major or raft::col_major (or one of their aliases)");
  RAFT_EXPECTS(input.extent(1) == output.extent(0), "Size mismatch between input and output");
  raft::detail::rmi::reduce(&handle, resource::get_cuda_stream(handle), output.data_handle(),
                            input.data_handle(), (std::int64_t)input.extent(0),
                            (std::int64_t)input.extent(1), is_row_major, false, raft::detail::rmi::zero<value_t>(), false,
                            raft::identity_op(), raft::add_op(), raft::identity_op());
}

}  // namespace raft::stats
