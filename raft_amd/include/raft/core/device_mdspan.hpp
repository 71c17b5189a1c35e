// Device-memory views used in the reduction API's signatures
// (core/device_mdspan.hpp:75-98,152-226 in the reference).
#pragma once

#include <raft/core/mdspan.hpp>

namespace raft {

template <typename ElementType, typename Extents, typename LayoutPolicy = layout_c_contiguous>
using device_mdspan = mdspan<ElementType, Extents, LayoutPolicy>;

template <typename ElementType, typename IndexType = int>
using device_scalar_view = device_mdspan<ElementType, scalar_extent<IndexType>>;

template <typename ElementType, typename IndexType = int, typename LayoutPolicy = layout_c_contiguous>
using device_vector_view = device_mdspan<ElementType, vector_extent<IndexType>, LayoutPolicy>;

template <typename ElementType, typename IndexType = int, typename LayoutPolicy = layout_c_contiguous>
using device_matrix_view = device_mdspan<ElementType, matrix_extent<IndexType>, LayoutPolicy>;

template <typename ElementType, typename IndexType = int>
constexpr auto make_device_scalar_view(ElementType* ptr)
{
  return device_scalar_view<ElementType, IndexType>{ptr, scalar_extent<IndexType>{}};
}

template <typename ElementType, typename IndexType = int, typename LayoutPolicy = layout_c_contiguous>
constexpr auto make_device_matrix_view(ElementType* ptr, IndexType n_rows, IndexType n_cols)
{
  return device_matrix_view<ElementType, IndexType, LayoutPolicy>{
    ptr, matrix_extent<IndexType>{n_rows, n_cols}};
}

// A matrix whose leading dimension may exceed its row (row-major) or column
// (column-major) length; stride <= 0 means "contiguous".
template <typename ElementType, typename IndexType, typename LayoutPolicy = layout_c_contiguous>
constexpr auto make_device_strided_matrix_view(ElementType* ptr,
                                               IndexType n_rows,
                                               IndexType n_cols,
                                               IndexType stride)
{
  constexpr bool rm = std::is_same_v<LayoutPolicy, layout_c_contiguous>;
  static_assert(rm || std::is_same_v<LayoutPolicy, layout_f_contiguous>,
                "Unsupported layout policy for strided matrix view");
  const IndexType s0 = rm ? (stride > 0 ? stride : n_cols) : 1;
  const IndexType s1 = rm ? 1 : (stride > 0 ? stride : n_rows);
  return device_matrix_view<ElementType, IndexType, layout_stride>{
    ptr, matrix_extent<IndexType>{n_rows, n_cols}, {s0, s1}};
}

template <typename ElementType, typename IndexType = int, typename LayoutPolicy = layout_c_contiguous>
constexpr auto make_device_vector_view(ElementType* ptr, IndexType n)
{
  return device_vector_view<ElementType, IndexType, LayoutPolicy>{ptr, n};
}

}  // namespace raft
