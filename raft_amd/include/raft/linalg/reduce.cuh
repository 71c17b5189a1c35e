// raft::linalg::reduce: row- or column-wise reduction of a row- or column-major
// matrix with fused main_op / reduce_op / final_op (linalg/reduce.cuh:55-76,140-180
// in the reference).  A sum (add_op) is compensated: it is accumulated so that it
// agrees with an fp64 evaluation to well below the output type's rounding.
#pragma once

#include <raft/core/device_mdspan.hpp>
#include <raft/core/operators.hpp>
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/core/types.hpp>
#include <raft/linalg/detail/rmi_bridge.hpp>
#include <raft/linalg/linalg_types.hpp>
#include <raft/util/input_validation.hpp>

namespace raft::linalg {

// Pointer form.  data: N rows x D columns; dots: N outputs (alongRows) or D.
template <bool rowMajor,
          bool alongRows,
          typename InType,
          typename OutType      = InType,
          typename IdxType      = int,
          typename MainLambda   = raft::identity_op,
          typename ReduceLambda = raft::add_op,
          typename FinalLambda  = raft::identity_op>
void reduce(OutType* dots,
            const InType* data,
            IdxType D,
            IdxType N,
            OutType init,
            hipStream_t stream,
            bool inplace           = false,
            MainLambda main_op     = raft::identity_op(),
            ReduceLambda reduce_op = raft::add_op(),
            FinalLambda final_op   = raft::identity_op())
{
  raft::detail::rmi::reduce(nullptr, stream, dots, data, (std::int64_t)N, (std::int64_t)D,
                            rowMajor, alongRows, init, inplace, main_op, reduce_op, final_op);
}

// mdspan form.  Apply::ALONG_ROWS gives one output per row, ALONG_COLUMNS one per
// column.  `init` must be reduce_op's neutral element.
template <Apply apply,
          typename InElementType,
          typename LayoutPolicy,
          typename OutElementType = InElementType,
          typename IdxType        = std::uint32_t,
          typename MainLambda     = raft::identity_op,
          typename ReduceLambda   = raft::add_op,
          typename FinalLambda    = raft::identity_op>
void reduce(raft::resources const& handle,
            raft::device_matrix_view<const InElementType, IdxType, LayoutPolicy> data,
            raft::device_vector_view<OutElementType, IdxType> dots,
            OutElementType init,
            bool inplace           = false,
            MainLambda main_op     = raft::identity_op(),
            ReduceLambda reduce_op = raft::add_op(),
            FinalLambda final_op   = raft::identity_op())
{
  RAFT_EXPECTS(raft::is_row_or_column_major(data), "Input must be contiguous");
  constexpr bool along_rows = apply == Apply::ALONG_ROWS;
  const bool row_major      = raft::is_row_major(data);
  if constexpr (along_rows) {
    RAFT_EXPECTS(static_cast<IdxType>(dots.size()) == data.extent(0),
                 "Output should be equal to number of rows in Input");
  } else {
    RAFT_EXPECTS(static_cast<IdxType>(dots.size()) == data.extent(1),
                 "Output should be equal to number of columns in Input");
  }
  if constexpr (std::is_same_v<LayoutPolicy, raft::layout_stride>) {
    RAFT_EXPECTS(data.is_exhaustive(), "Input must be contiguous");
  }
  raft::detail::rmi::reduce(&handle, resource::get_cuda_stream(handle), dots.data_handle(),
                            data.data_handle(), (std::int64_t)data.extent(0),
                            (std::int64_t)data.extent(1), row_major, along_rows, init, inplace,
                            main_op, reduce_op, final_op);
}

}  // namespace raft::linalg
