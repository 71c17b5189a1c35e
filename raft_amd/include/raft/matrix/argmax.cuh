// Index of the maximum of every row of a row-major matrix, lowest index on ties
// (matrix/argmax.cuh:27-39, matrix/detail/math.cuh:291-352 in the reference): a
// key-value arg-reduction started from (0, -inf) whose key alone is written.
#pragma once

#include <limits>

#include <raft/core/device_mdspan.hpp>
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/linalg/detail/rmi_bridge.hpp>

namespace raft::matrix {

template <typename math_t, typename idx_t, typename matrix_idx_t>
void argmax(raft::resources const& handle,
            raft::device_matrix_view<const math_t, matrix_idx_t, row_major> in,
            raft::device_vector_view<idx_t, matrix_idx_t> out)
{
  RAFT_EXPECTS(out.extent(0) == in.extent(0),
               "Size of output vector must equal number of rows in input matrix.");
  static_assert(std::is_integral_v<idx_t> && (sizeof(idx_t) == 4 || sizeof(idx_t) == 8),
                "argmax: the index type must be a 32- or 64-bit integer");
  using key_t = std::conditional_t<sizeof(idx_t) == 4, std::int32_t, std::int64_t>;
  using kvp_t = raft::KeyValuePair<key_t, math_t>;
  // the accumulator is a key-value pair; RMI_FIN_KEY stores only its key, as idx_t
  raft::detail::rmi::reduce(&handle, resource::get_cuda_stream(handle),
                            reinterpret_cast<kvp_t*>(out.data_handle()), in.data_handle(),
                            (std::int64_t)in.extent(0), (std::int64_t)in.extent(1), true, true,
                            kvp_t(0, -std::numeric_limits<math_t>::infinity()), false,
                            raft::value_to_kvp_op<key_t>(), raft::argmax_op(), raft::key_op(), -1,
                            0.0, 0.0, nullptr, sizeof(idx_t) == 4 ? RMI_I32 : RMI_I64);
}

}  // namespace raft::matrix
