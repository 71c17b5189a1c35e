// Row and column norms as functor triples over reduce (linalg/norm.cuh:45-148,
// linalg/detail/norm.cuh:23-61 in the reference): L1 = (abs, add), L2 = (sq, add),
// Linf = (abs, max), init 0, then the caller's fin_op (sqrt_op for a true L2 norm).
#pragma once

#include <raft/linalg/norm_types.hpp>
#include <raft/linalg/reduce.cuh>

namespace raft::linalg {
namespace detail {
template <NormType norm_type, bool rowMajor, bool alongRows, typename Type, typename OutType,
          typename IdxType, typename Lambda>
void norm_call(const resources* res, OutType* dots, const Type* data, IdxType D, IdxType N,
               hipStream_t stream, Lambda fin_op)
{
  static_assert(norm_type == L1Norm || norm_type == L2Norm || norm_type == LinfNorm,
                "Unsupported norm type");
  namespace b = raft::detail::rmi;
  if constexpr (norm_type == L1Norm) {
    b::reduce(res, stream, dots, data, (std::int64_t)N, (std::int64_t)D, rowMajor, alongRows,
              b::zero<OutType>(), false, raft::abs_op(), raft::add_op(), fin_op);
  } else if constexpr (norm_type == L2Norm) {
    b::reduce(res, stream, dots, data, (std::int64_t)N, (std::int64_t)D, rowMajor, alongRows,
              b::zero<OutType>(), false, raft::sq_op(), raft::add_op(), fin_op);
  } else {
    b::reduce(res, stream, dots, data, (std::int64_t)N, (std::int64_t)D, rowMajor, alongRows,
              b::zero<OutType>(), false, raft::abs_op(), raft::max_op(), fin_op);
  }
}
}  // namespace detail

// data: N rows x D columns.  rowNorm writes N values, colNorm writes D.
template <NormType norm_type, bool rowMajor, typename Type, typename IdxType = int,
          typename Lambda = raft::identity_op, typename OutType = Type>
void rowNorm(OutType* dots, const Type* data, IdxType D, IdxType N, hipStream_t stream,
             Lambda fin_op = raft::identity_op())
{
  detail::norm_call<norm_type, rowMajor, true>(nullptr, dots, data, D, N, stream, fin_op);
}

template <NormType norm_type, bool rowMajor, typename Type, typename IdxType = int,
          typename Lambda = raft::identity_op, typename OutType = Type>
void colNorm(OutType* dots, const Type* data, IdxType D, IdxType N, hipStream_t stream,
             Lambda fin_op = raft::identity_op())
{
  detail::norm_call<norm_type, rowMajor, false>(nullptr, dots, data, D, N, stream, fin_op);
}

template <NormType norm_type,
          raft::Apply apply,
          typename ElementType,
          typename OutputType,
          typename LayoutPolicy,
          typename IndexType,
          typename Lambda = raft::identity_op>
void norm(raft::resources const& handle,
          raft::device_matrix_view<const ElementType, IndexType, LayoutPolicy> in,
          raft::device_vector_view<OutputType, IndexType> out,
          Lambda fin_op = raft::identity_op())
{
  RAFT_EXPECTS(raft::is_row_or_column_major(in), "Input must be contiguous");
  constexpr bool row_major  = std::is_same_v<LayoutPolicy, raft::row_major>;
  constexpr bool along_rows = apply == raft::Apply::ALONG_ROWS;
  static_assert(row_major || std::is_same_v<LayoutPolicy, raft::col_major>,
                "norm: layout must be row_major or col_major");
  if constexpr (along_rows) {
    RAFT_EXPECTS(static_cast<IndexType>(out.size()) == in.extent(0),
                 "Output should be equal to number of rows in Input");
  } else {
    RAFT_EXPECTS(static_cast<IndexType>(out.size()) == in.extent(1),
                 "Output should be equal to number of columns in Input");
  }
  detail::norm_call<norm_type, row_major, along_rows>(&handle, out.data_handle(),
                                                      in.data_handle(), in.extent(1),
                                                      in.extent(0),
                                                      resource::get_cuda_stream(handle), fin_op);
}

}  // namespace raft::linalg
