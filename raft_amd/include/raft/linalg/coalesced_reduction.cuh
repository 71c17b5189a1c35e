// Reduction along the contiguous dimension (linalg/coalesced_reduction.cuh in the
// reference): dots[i] = final_op(reduce_op-fold over j of main_op(data[i*D + j], j)).
#pragma once

#include <raft/core/device_mdspan.hpp>
#include <raft/core/operators.hpp>
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/linalg/detail/rmi_bridge.hpp>

namespace raft::linalg {

// data: N rows of D contiguous elements; dots: N outputs.
template <typename InType,
          typename OutType      = InType,
          typename IdxType      = int,
          typename MainLambda   = raft::identity_op,
          typename ReduceLambda = raft::add_op,
          typename FinalLambda  = raft::identity_op>
void coalescedReduction(OutType* dots,
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
  raft::detail::rmi::reduce(nullptr, stream, dots, data, (std::int64_t)N, (std::int64_t)D, true,
                            true, init, inplace, main_op, reduce_op, final_op);
}

template <typename InValueType,
          typename LayoutPolicy,
          typename OutValueType,
          typename IdxType,
          typename MainLambda   = raft::identity_op,
          typename ReduceLambda = raft::add_op,
          typename FinalLambda  = raft::identity_op>
void coalesced_reduction(raft::resources const& handle,
                         raft::device_matrix_view<const InValueType, IdxType, LayoutPolicy> data,
                         raft::device_vector_view<OutValueType, IdxType> dots,
                         OutValueType init,
                         bool inplace           = false,
                         MainLambda main_op     = raft::identity_op(),
                         ReduceLambda reduce_op = raft::add_op(),
                         FinalLambda final_op   = raft::identity_op())
{
  constexpr bool rm = std::is_same_v<LayoutPolicy, raft::row_major>;
  static_assert(rm || std::is_same_v<LayoutPolicy, raft::col_major>,
                "coalesced_reduction: layout must be row_major or col_major");
  if constexpr (rm) {
    RAFT_EXPECTS(static_cast<IdxType>(dots.size()) == data.extent(0),
                 "Output should be equal to number of rows in Input");
  } else {
    RAFT_EXPECTS(static_cast<IdxType>(dots.size()) == data.extent(1),
                 "Output should be equal to number of columns in Input");
  }
  // row-major: one output per row; column-major: one per column -- in both cases
  // the fold runs along the contiguous dimension
  raft::detail::rmi::reduce(&handle, resource::get_cuda_stream(handle), dots.data_handle(),
                            data.data_handle(), (std::int64_t)data.extent(0),
                            (std::int64_t)data.extent(1), rm, rm, init, inplace, main_op,
                            reduce_op, final_op);
}

}  // namespace raft::linalg
