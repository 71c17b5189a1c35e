// raft::stats::cov (stats/cov.cuh:38-50 pointer form, :77-106 mdspan form; stats/detail/cov.cuh:38-66
// in the reference): covariance matrix of the columns of `data` around the mean vector `mu`,
// normalised by N - 1 (sample) or N.  As in the reference the call mean-centres `data` in
// place ("this will get mean-centered at the end!") and only the stable variant exists:
// stable == false raises, like the reference's ASSERT (stats/detail/cov.cuh:61-63).
//
// One fused pass on the matrix cores (rmi_cov in the reduction library) in place of the
// reference's meanCenter launch followed by a cuBLAS GEMM; plain C++, no device code in the
// caller's translation unit.
#pragma once

#include <cstddef>
#include <type_traits>

#include <raft/core/device_mdspan.hpp>
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/linalg/detail/rmi_bridge.hpp>

namespace raft::stats {
namespace detail {
template <bool rowMajor, typename Type>
void cov(const resources* res, Type* covar, Type* data, const Type* mu, std::size_t D,
         std::size_t N, bool sample, bool stable, hipStream_t stream)
{
  static_assert(std::is_same_v<Type, float> || std::is_same_v<Type, double>,
                "cov: float and double data are offered (the reference's GEMM types)");
  ASSERT(stable, "cov: Implement stable=false case!");
  const int dtype  = raft::detail::rmi::dtype_of<Type>::value;
  const int layout = rowMajor ? RMI_ROW_MAJOR : RMI_COL_MAJOR;
  const size_t ws_bytes =
    rmi_cov_workspace_bytes(dtype, layout, (std::int64_t)N, (std::int64_t)D);
  raft::detail::rmi::workspace_lease ws(res, stream, ws_bytes);
  raft::detail::rmi::check(
    rmi_cov(dtype, layout, (std::int64_t)N, (std::int64_t)D, sample ? 1 : 0, RMI_COV_CENTER_DATA,
            data, mu, covar, ws.data(), ws.size(), stream),
    "rmi_cov");
}
}  // namespace detail

// data: N rows x D columns (mean-centred when the call returns); mu: D means; covar: D x D.
template <bool rowMajor, typename Type>
void cov(raft::resources const& handle,
         Type* covar,
         Type* data,
         const Type* mu,
         std::size_t D,
         std::size_t N,
         bool sample,
         bool stable,
         hipStream_t stream)
{
  detail::cov<rowMajor>(&handle, covar, data, mu, D, N, sample, stable, stream);
}

template <typename value_t, typename idx_t, typename layout_t>
void cov(raft::resources const& handle,
         raft::device_matrix_view<value_t, idx_t, layout_t> data,
         raft::device_vector_view<const value_t, idx_t> mu,
         raft::device_matrix_view<value_t, idx_t, layout_t> covar,
         bool sample,
         bool stable)
{
  static_assert(
    std::is_same_v<layout_t, raft::row_major> || std::is_same_v<layout_t, raft::col_major>,
    "Data layout not supported");
  RAFT_EXPECTS(data.extent(1) == covar.extent(0) && data.extent(1) == covar.extent(1),
               "Size mismatch");
  RAFT_EXPECTS(data.is_exhaustive(), "data must be contiguous");
  RAFT_EXPECTS(covar.is_exhaustive(), "covar must be contiguous");
  RAFT_EXPECTS(mu.is_exhaustive(), "mu must be contiguous");
  detail::cov<std::is_same_v<layout_t, raft::row_major>>(
    &handle, covar.data_handle(), data.data_handle(), mu.data_handle(),
    (std::size_t)data.extent(1), (std::size_t)data.extent(0), sample, stable,
    resource::get_cuda_stream(handle));
}

}  // namespace raft::stats
