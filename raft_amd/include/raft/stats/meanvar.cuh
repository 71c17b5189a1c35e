// Mean and variance of every column in one pass over the data
// (stats/meanvar.cuh:38-98, stats/detail/meanvar.cuh:187-236 in the reference):
// mean[j] = sum_i data[i, j] / N, var[j] = sum_i (data[i, j] - mean[j])^2 /
// max(1, sample ? N - 1 : N).  One read of the matrix instead of the two that
// mean followed by vars takes.
#pragma once

#include <type_traits>

#include <raft/core/device_mdspan.hpp>
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/linalg/detail/rmi_bridge.hpp>

namespace raft::stats {
namespace detail {
template <typename T, typename I>
void meanvar(const resources* res, T* mean, T* var, const T* data, I D, I N, bool sample,
             bool rowMajor, hipStream_t stream)
{
  static_assert(std::is_same_v<T, float> || std::is_same_v<T, double> || std::is_same_v<T, __half> ||
                  std::is_same_v<T, raft::bfloat16_t>,
                "meanvar: float, double, half and bfloat16 data are offered");
  const int dtype  = raft::detail::rmi::dtype_of<T>::value;
  const int layout = rowMajor ? RMI_ROW_MAJOR : RMI_COL_MAJOR;
  const size_t ws_bytes =
    rmi_meanvar_workspace_bytes(dtype, layout, (std::int64_t)N, (std::int64_t)D);
  raft::detail::rmi::workspace_lease ws(res, stream, ws_bytes);
  raft::detail::rmi::check(rmi_meanvar(dtype, layout, (std::int64_t)N, (std::int64_t)D,
                                       sample ? 1 : 0, data, mean, var, ws.data(), ws.size(),
                                       stream),
                           "rmi_meanvar");
}
}  // namespace detail

// data: N rows x D columns; mean, var: D values each.
template <typename Type, typename IdxType = int>
void meanvar(Type* mean,
             Type* var,
             const Type* data,
             IdxType D,
             IdxType N,
             bool sample,
             bool rowMajor,
             hipStream_t stream)
{
  detail::meanvar(nullptr, mean, var, data, D, N, sample, rowMajor, stream);
}

template <typename value_t, typename idx_t, typename layout_t>
void meanvar(raft::resources const& handle,
             raft::device_matrix_view<const value_t, idx_t, layout_t> data,
             raft::device_vector_view<value_t, idx_t> mean,
             raft::device_vector_view<value_t, idx_t> var,
             bool sample)
{
  static_assert(
    std::is_same_v<layout_t, raft::row_major> || std::is_same_v<layout_t, raft::col_major>,
    "Data layout not supported");
  RAFT_EXPECTS(data.extent(1) == var.extent(0), "Size mismatch between data and var");
  RAFT_EXPECTS(mean.size() == var.size(), "Size mismatch between mean and var");
  RAFT_EXPECTS(mean.is_exhaustive(), "mean must be contiguous");
  RAFT_EXPECTS(var.is_exhaustive(), "var must be contiguous");
  RAFT_EXPECTS(data.is_exhaustive(), "data must be contiguous");
  detail::meanvar(&handle, mean.data_handle(), var.data_handle(), data.data_handle(),
                  data.extent(1), data.extent(0), sample,
                  std::is_same_v<layout_t, raft::row_major>, resource::get_cuda_stream(handle));
}

}  // namespace raft::stats
