// Column means (stats/mean.cuh:36-157, stats/detail/mean.cuh:19-57 in the
// reference): mu[j] = (sum over rows of data[i, j]) * ratio with ratio = 1/N rounded
// to the output type first, fused into the reduction's epilogue.
#pragma once

#include <type_traits>

#include <raft/core/device_mdspan.hpp>
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/linalg/detail/rmi_bridge.hpp>

namespace raft::stats {
namespace detail {
template <typename OutType>
double rounded_ratio(double denom)
{
  if constexpr (std::is_same_v<OutType, __half>) {
    // OutType(1) / OutType(N) in half arithmetic
    const float d = __half2float(__float2half((float)denom));
    return (double)__half2float(__float2half(1.0f / d));
  } else {
    return (double)(OutType(1) / OutType(denom));
  }
}

template <bool rowMajor, typename OutType, typename InType, typename IdxType>
void mean_call(const resources* res, OutType* mu, const InType* data, IdxType D, IdxType N,
               double denom, hipStream_t stream)
{
  raft::detail::rmi::reduce(res, stream, mu, data, (std::int64_t)N, (std::int64_t)D, rowMajor,
                            false, raft::detail::rmi::zero<OutType>(), false, raft::identity_op(), raft::add_op(),
                            raft::identity_op(), RMI_FIN_MUL_CONST,
                            rounded_ratio<OutType>(denom));
}
}  // namespace detail

// data: N rows x D columns; mu: D means.
template <bool rowMajor, typename Type, typename IdxType = int>
void mean(Type* mu, const Type* data, IdxType D, IdxType N, hipStream_t stream)
{
  detail::mean_call<rowMajor>(nullptr, mu, data, D, N, (double)N, stream);
}

template <bool rowMajor, typename Type, typename IdxType = int>
[[deprecated("'sample' parameter deprecated")]] void mean(
  Type* mu, const Type* data, IdxType D, IdxType N, bool sample, hipStream_t stream)
{
  detail::mean_call<rowMajor>(nullptr, mu, data, D, N, sample ? (double)(N - 1) : (double)N,
                              stream);
}

template <typename in_value_t, typename out_value_t, typename idx_t, typename layout_t>
void mean(raft::resources const& handle,
          raft::device_matrix_view<const in_value_t, idx_t, layout_t> data,
          raft::device_vector_view<out_value_t, idx_t> mu)
{
  static_assert(
    std::is_same_v<layout_t, raft::row_major> || std::is_same_v<layout_t, raft::col_major>,
    "Data layout not supported");
  RAFT_EXPECTS(data.extent(1) == mu.extent(0), "Size mismatch between data and mu");
  RAFT_EXPECTS(mu.is_exhaustive(), "mu must be contiguous");
  RAFT_EXPECTS(data.is_exhaustive(), "data must be contiguous");
  detail::mean_call<std::is_same_v<layout_t, raft::row_major>>(
    &handle, mu.data_handle(), data.data_handle(), data.extent(1), data.extent(0),
    (double)data.extent(0), resource::get_cuda_stream(handle));
}

template <typename value_t, typename idx_t, typename layout_t>
[[deprecated("'sample' parameter deprecated")]] void mean(
  raft::resources const& handle,
  raft::device_matrix_view<const value_t, idx_t, layout_t> data,
  raft::device_vector_view<value_t, idx_t> mu,
  bool sample)
{
  static_assert(
    std::is_same_v<layout_t, raft::row_major> || std::is_same_v<layout_t, raft::col_major>,
    "Data layout not supported");
  RAFT_EXPECTS(data.extent(1) == mu.extent(0), "Size mismatch between data and mu");
  RAFT_EXPECTS(mu.is_exhaustive(), "mu must be contiguous");
  RAFT_EXPECTS(data.is_exhaustive(), "data must be contiguous");
  const double n = (double)data.extent(0);
  detail::mean_call<std::is_same_v<layout_t, raft::row_major>>(
    &handle, mu.data_handle(), data.data_handle(), data.extent(1), data.extent(0),
    sample ? n - 1 : n, resource::get_cuda_stream(handle));
}

}  // namespace raft::stats
