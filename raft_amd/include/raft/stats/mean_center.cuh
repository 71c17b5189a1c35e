// raft::stats::meanCenter / meanAdd / mean_center / mean_add (stats/mean_center.cuh:31-140,
// stats/detail/mean_center.cuh:30-60 in the reference): out = data -/+ mu, the mean vector
// broadcast along the rows (one mean per column) or along the columns.  Built on
// matrix_vector_op: compile with hipcc.
#pragma once

#include <type_traits>

#include <raft/core/device_mdspan.hpp>
#include <raft/core/operators.hpp>
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/linalg/matrix_vector_op.cuh>

namespace raft::stats {

template <bool rowMajor, bool bcastAlongRows, typename Type, typename IdxType = int>
void meanCenter(Type* out, const Type* data, const Type* mu, IdxType D, IdxType N, hipStream_t stream)
{
  raft::linalg::matrixVectorOp<rowMajor, bcastAlongRows>(out, data, mu, D, N, raft::sub_op{}, stream);
}

template <bool rowMajor, bool bcastAlongRows, typename Type, typename IdxType = int>
void meanAdd(Type* out, const Type* data, const Type* mu, IdxType D, IdxType N, hipStream_t stream)
{
  raft::linalg::matrixVectorOp<rowMajor, bcastAlongRows>(out, data, mu, D, N, raft::add_op{}, stream);
}

template <raft::Apply apply, typename value_t, typename idx_t, typename layout_t>
void mean_center(raft::resources const& handle,
                 raft::device_matrix_view<const value_t, idx_t, layout_t> data,
                 raft::device_vector_view<const value_t, idx_t> mu,
                 raft::device_matrix_view<value_t, idx_t, layout_t> out)
{
  static_assert(std::is_same_v<layout_t, raft::row_major> || std::is_same_v<layout_t, raft::col_major>,
                "Data layout not supported");
  const auto mean_vec_size = apply == raft::Apply::ALONG_ROWS ? data.extent(1) : data.extent(0);
  RAFT_EXPECTS(out.extent(0) == data.extent(0) && out.extent(1) == data.extent(1), "Size mismatch");
  RAFT_EXPECTS(mean_vec_size == mu.extent(0), "Size mismatch between data and mu");
  RAFT_EXPECTS(out.is_exhaustive(), "out must be contiguous");
  RAFT_EXPECTS(data.is_exhaustive(), "data must be contiguous");
  meanCenter<std::is_same_v<layout_t, raft::row_major>, apply == raft::Apply::ALONG_ROWS, value_t, idx_t>(
    out.data_handle(), data.data_handle(), mu.data_handle(), data.extent(1), data.extent(0),
    resource::get_cuda_stream(handle));
}

template <raft::Apply apply, typename value_t, typename idx_t, typename layout_t>
void mean_add(raft::resources const& handle,
              raft::device_matrix_view<const value_t, idx_t, layout_t> data,
              raft::device_vector_view<const value_t, idx_t> mu,
              raft::device_matrix_view<value_t, idx_t, layout_t> out)
{
  static_assert(std::is_same_v<layout_t, raft::row_major> || std::is_same_v<layout_t, raft::col_major>,
                "Data layout not supported");
  const auto mean_vec_size = apply == raft::Apply::ALONG_ROWS ? data.extent(1) : data.extent(0);
  RAFT_EXPECTS(out.extent(0) == data.extent(0) && out.extent(1) == data.extent(1), "Size mismatch");
  RAFT_EXPECTS(mean_vec_size == mu.extent(0), "Size mismatch between data and mu");
  RAFT_EXPECTS(out.is_exhaustive(), "out must be contiguous");
  RAFT_EXPECTS(data.is_exhaustive(), "data must be contiguous");
  meanAdd<std::is_same_v<layout_t, raft::row_major>, apply == raft::Apply::ALONG_ROWS, value_t, idx_t>(
    out.data_handle(), data.data_handle(), mu.data_handle(), data.extent(1), data.extent(0),
    resource::get_cuda_stream(handle));
}

}  // namespace raft::stats
