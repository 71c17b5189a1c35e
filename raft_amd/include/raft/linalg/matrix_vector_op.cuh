// raft::linalg::matrixVectorOp / matrix_vector_op (linalg/matrix_vector_op.cuh:48-233 in
// the reference): out[i][j] = op(matrix[i][j], vec[j]) when the vector is broadcast along the
// rows (one entry per column), op(matrix[i][j], vec[i]) otherwise; one or two vectors.
// Header templates over the caller's functor: compile with hipcc.
#pragma once

#include <type_traits>

#include <raft/core/device_mdspan.hpp>
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/linalg/detail/matrix_vector_op.cuh>
#include <raft/linalg/linalg_types.hpp>

namespace raft::linalg {

template <bool rowMajor, bool bcastAlongRows, typename MatT, typename Lambda, typename VecT,
          typename IdxType = int>
void matrixVectorOp(MatT* out, const MatT* matrix, const VecT* vec, IdxType D, IdxType N, Lambda op,
                    hipStream_t stream)
{
  detail::matrixVectorOpImpl<rowMajor, bcastAlongRows, false>(out, matrix, D, N, op, stream, vec,
                                                              static_cast<const VecT*>(nullptr));
}

template <bool rowMajor, bool bcastAlongRows, typename MatT, typename Lambda, typename Vec1T,
          typename Vec2T, typename IdxType = int>
void matrixVectorOp(MatT* out, const MatT* matrix, const Vec1T* vec1, const Vec2T* vec2, IdxType D,
                    IdxType N, Lambda op, hipStream_t stream)
{
  detail::matrixVectorOpImpl<rowMajor, bcastAlongRows, true>(out, matrix, D, N, op, stream, vec1, vec2);
}

template <Apply apply, typename MatValueType, typename VecValueType, typename LayoutPolicy,
          typename Lambda, typename IndexType>
void matrix_vector_op(raft::resources const& handle,
                      raft::device_matrix_view<const MatValueType, IndexType, LayoutPolicy> matrix,
                      raft::device_vector_view<const VecValueType, IndexType> vec,
                      raft::device_matrix_view<MatValueType, IndexType, LayoutPolicy> out, Lambda op)
{
  static_assert(std::is_same_v<LayoutPolicy, raft::row_major> ||
                  std::is_same_v<LayoutPolicy, raft::col_major>,
                "matrix_vector_op: row- or column-major matrices");
  RAFT_EXPECTS(matrix.is_exhaustive(), "Input must be contiguous");
  RAFT_EXPECTS(out.is_exhaustive(), "Output must be contiguous");
  RAFT_EXPECTS(out.size() == matrix.size(), "Size mismatch between Output and Input");
  constexpr bool rowMajor       = std::is_same_v<LayoutPolicy, raft::row_major>;
  constexpr bool bcastAlongRows = apply == Apply::ALONG_ROWS;
  RAFT_EXPECTS((bcastAlongRows ? out.extent(1) : out.extent(0)) == static_cast<IndexType>(vec.size()),
               "Size mismatch between matrix and vector");
  matrixVectorOp<rowMajor, bcastAlongRows>(out.data_handle(), matrix.data_handle(),
                                           vec.data_handle(), out.extent(1), out.extent(0), op,
                                           resource::get_cuda_stream(handle));
}

template <Apply apply, typename MatValueType, typename Vec1ValueType, typename Vec2ValueType,
          typename LayoutPolicy, typename Lambda, typename IndexType>
void matrix_vector_op(raft::resources const& handle,
                      raft::device_matrix_view<const MatValueType, IndexType, LayoutPolicy> matrix,
                      raft::device_vector_view<const Vec1ValueType, IndexType> vec1,
                      raft::device_vector_view<const Vec2ValueType, IndexType> vec2,
                      raft::device_matrix_view<MatValueType, IndexType, LayoutPolicy> out, Lambda op)
{
  static_assert(std::is_same_v<LayoutPolicy, raft::row_major> ||
                  std::is_same_v<LayoutPolicy, raft::col_major>,
                "matrix_vector_op: row- or column-major matrices");
  RAFT_EXPECTS(matrix.is_exhaustive(), "Input must be contiguous");
  RAFT_EXPECTS(out.is_exhaustive(), "Output must be contiguous");
  RAFT_EXPECTS(out.size() == matrix.size(), "Size mismatch between Output and Input");
  constexpr bool rowMajor       = std::is_same_v<LayoutPolicy, raft::row_major>;
  constexpr bool bcastAlongRows = apply == Apply::ALONG_ROWS;
  const IndexType want          = bcastAlongRows ? out.extent(1) : out.extent(0);
  RAFT_EXPECTS(want == static_cast<IndexType>(vec1.size()), "Size mismatch between matrix and vector");
  RAFT_EXPECTS(want == static_cast<IndexType>(vec2.size()), "Size mismatch between matrix and vector");
  matrixVectorOp<rowMajor, bcastAlongRows>(out.data_handle(), matrix.data_handle(),
                                           vec1.data_handle(), vec2.data_handle(), out.extent(1),
                                           out.extent(0), op, resource::get_cuda_stream(handle));
}

}  // namespace raft::linalg
