// Row normalisation (linalg/normalize.cuh:48-110 in the reference): every row is
// divided by its norm; rows whose norm is <= eps are not written.  The norm and the
// scaling are one fused kernel of the reduction library.
#pragma once

#include <raft/core/device_mdspan.hpp>
#include <raft/core/operators.hpp>
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/linalg/detail/rmi_bridge.hpp>
#include <raft/linalg/norm_types.hpp>
#include <raft/util/input_validation.hpp>

namespace raft::linalg {

// norm_i = fin_op(reduce_op-fold of main_op(in[i, j]) starting from init)
template <typename ElementType,
          typename IndexType,
          typename MainLambda,
          typename ReduceLambda,
          typename FinalLambda>
void row_normalize(raft::resources const& handle,
                   raft::device_matrix_view<const ElementType, IndexType, row_major> in,
                   raft::device_matrix_view<ElementType, IndexType, row_major> out,
                   ElementType init,
                   MainLambda main_op,
                   ReduceLambda reduce_op,
                   FinalLambda fin_op,
                   ElementType eps = ElementType(1e-8))
{
  RAFT_EXPECTS(raft::is_row_or_column_major(in), "Input must be contiguous");
  RAFT_EXPECTS(raft::is_row_or_column_major(out), "Output must be contiguous");
  RAFT_EXPECTS(in.extent(0) == out.extent(0),
               "The number of rows of the input and output should be equal");
  RAFT_EXPECTS(in.extent(1) == out.extent(1),
               "The number of columns of the input and output should be equal");
  namespace b = raft::detail::rmi;
  static_assert(b::main_tag<MainLambda>::value >= 0 && b::reduce_tag<ReduceLambda>::value >= 0 &&
                  (std::is_same_v<FinalLambda, raft::identity_op> ||
                   std::is_same_v<FinalLambda, raft::sqrt_op>),
                "row_normalize: main_op must be identity_op / sq_op / abs_op, reduce_op add_op / "
                "max_op / min_op and fin_op identity_op or sqrt_op");
  (void)main_op;
  (void)reduce_op;
  (void)fin_op;
  rmi_reduce_desc d{};
  d.in_dtype  = b::dtype<ElementType>();
  d.out_dtype = d.in_dtype;
  d.layout    = RMI_ROW_MAJOR;
  d.apply     = RMI_ALONG_ROWS;
  d.n_rows    = (std::int64_t)in.extent(0);
  d.n_cols    = (std::int64_t)in.extent(1);
  d.main_op   = b::main_tag<MainLambda>::value;
  d.reduce_op = b::reduce_tag<ReduceLambda>::value;
  d.final_op  = b::final_tag<FinalLambda>::value;
  d.init      = b::make_init(init);
  b::check(rmi_row_normalize(&d, in.data_handle(), out.data_handle(), b::to_double(eps),
                             resource::get_cuda_stream(handle)),
           "rmi_row_normalize");
}

// L1: x / sum|x|, L2: x / sqrt(sum x^2), Linf: x / max|x|
template <NormType norm_type, typename ElementType, typename IndexType>
void row_normalize(raft::resources const& handle,
                   raft::device_matrix_view<const ElementType, IndexType, row_major> in,
                   raft::device_matrix_view<ElementType, IndexType, row_major> out,
                   ElementType eps = ElementType(1e-8))
{
  static_assert(norm_type == L1Norm || norm_type == L2Norm || norm_type == LinfNorm,
                "Unsupported norm type");
  if constexpr (norm_type == L1Norm) {
    row_normalize(
      handle, in, out, ElementType(0), raft::abs_op(), raft::add_op(), raft::identity_op(), eps);
  } else if constexpr (norm_type == L2Norm) {
    row_normalize(
      handle, in, out, ElementType(0), raft::sq_op(), raft::add_op(), raft::sqrt_op(), eps);
  } else {
    row_normalize(
      handle, in, out, ElementType(0), raft::abs_op(), raft::max_op(), raft::identity_op(), eps);
  }
}

}  // namespace raft::linalg
