// Column standard deviation and variance given the column means
// (stats/stddev.cuh:37-167, stats/detail/stddev.cuh:37-102 in the reference):
//   sum_sq[j] = sum over rows of data[i, j]^2
//   var[j]    = | sum_sq[j] * ratio - mu[j]^2 * ratio_mean |,   stddev = sqrt(var)
//   ratio = 1/(N-1) (sample) or 1/N, ratio_mean = sample ? ratio * N : 1,
// every step in the element type.  The reference launches a fill, a reduction and
// an elementwise epilogue; here the epilogue is the reduction's final_op.
#pragma once

#include <raft/core/device_mdspan.hpp>
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/linalg/detail/rmi_bridge.hpp>

namespace raft::stats {
namespace detail {
template <bool rowMajor, typename Type, typename IdxType>
void second_moment_call(const resources* res, Type* out, const Type* data, const Type* mu,
                        IdxType D, IdxType N, bool sample, bool take_sqrt, hipStream_t stream)
{
  const Type ratio      = Type(1) / (sample ? Type(N - 1) : Type(N));
  const Type ratio_mean = sample ? ratio * Type(N) : Type(1);
  raft::detail::rmi::reduce(res, stream, out, data, (std::int64_t)N, (std::int64_t)D, rowMajor,
                            false, Type(0), false, raft::sq_op(), raft::add_op(),
                            raft::identity_op(),
                            take_sqrt ? RMI_FIN_STDDEV_FROM_SUMSQ : RMI_FIN_VAR_FROM_SUMSQ,
                            (double)ratio, (double)ratio_mean, mu);
}
}  // namespace detail

template <bool rowMajor, typename Type, typename IdxType = int>
void stddev(Type* std, const Type* data, const Type* mu, IdxType D, IdxType N, bool sample,
            hipStream_t stream)
{
  detail::second_moment_call<rowMajor>(nullptr, std, data, mu, D, N, sample, true, stream);
}

template <bool rowMajor, typename Type, typename IdxType = int>
void vars(Type* var, const Type* data, const Type* mu, IdxType D, IdxType N, bool sample,
          hipStream_t stream)
{
  detail::second_moment_call<rowMajor>(nullptr, var, data, mu, D, N, sample, false, stream);
}

template <typename value_t, typename idx_t, typename layout_t>
void stddev(raft::resources const& handle,
            raft::device_matrix_view<const value_t, idx_t, layout_t> data,
            raft::device_vector_view<const value_t, idx_t> mu,
            raft::device_vector_view<value_t, idx_t> std,
            bool sample)
{
  constexpr bool is_row_major = std::is_same_v<layout_t, raft::row_major>;
  static_assert(is_row_major || std::is_same_v<layout_t, raft::col_major>,
                "stddev: Layout must be either "
                "raft::row_major or raft::col_major (or one of their aliases)");
  RAFT_EXPECTS(mu.size() == std.size(), "Size mismatch between mu and std");
  RAFT_EXPECTS(mu.extent(0) == data.extent(1), "Size mismatch between data and mu");
  detail::second_moment_call<is_row_major>(&handle, std.data_handle(), data.data_handle(),
                                           mu.data_handle(), data.extent(1), data.extent(0),
                                           sample, true, resource::get_cuda_stream(handle));
}

template <typename value_t, typename idx_t, typename layout_t>
void vars(raft::resources const& handle,
          raft::device_matrix_view<const value_t, idx_t, layout_t> data,
          raft::device_vector_view<const value_t, idx_t> mu,
          raft::device_vector_view<value_t, idx_t> var,
          bool sample)
{
  constexpr bool is_row_major = std::is_same_v<layout_t, raft::row_major>;
  static_assert(is_row_major || std::is_same_v<layout_t, raft::col_major>,
                "vars: Layout must be either "
                "raft::row_major or raft::col_major (or one of their aliases)");
  RAFT_EXPECTS(mu.size() == var.size(), "Size mismatch between mu and std");
  RAFT_EXPECTS(mu.extent(0) == data.extent(1), "Size mismatch between data and mu");
  detail::second_moment_call<is_row_major>(&handle, var.data_handle(), data.data_handle(),
                                           mu.data_handle(), data.extent(1), data.extent(0),
                                           sample, false, resource::get_cuda_stream(handle));
}

}  // namespace raft::stats
