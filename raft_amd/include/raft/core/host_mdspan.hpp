// Non-owning views of host memory (core/host_mdspan.hpp:117-199 in the reference).  Unlike
// the device views these can be indexed: operator() with one index per dimension, and
// operator[] for scalars and vectors.
#pragma once

#include <raft/core/mdspan_types.hpp>

namespace raft {

template <typename ElementType, typename Extents, typename LayoutPolicy = layout_c_contiguous>
class host_mdspan : public mdspan<ElementType, Extents, LayoutPolicy> {
  using base = mdspan<ElementType, Extents, LayoutPolicy>;

 public:
  using base::base;
  constexpr host_mdspan(const base& b) : base(b) {}
  template <typename... I>
  constexpr ElementType& operator()(I... idx) const
  {
    return this->data_handle()[this->offset(idx...)];
  }
  // a scalar view answers [0], as the reference's does through its single-element extent
  template <typename I>
  constexpr ElementType& operator[](I i) const
  {
    if constexpr (Extents::rank() == 0) {
      return this->data_handle()[0];
    } else {
      static_assert(Extents::rank() == 1, "operator[] indexes scalars and vectors");
      return this->data_handle()[this->offset(i)];
    }
  }
};

template <typename ElementType, typename IndexType = int>
using host_scalar_view = host_mdspan<ElementType, scalar_extent<IndexType>>;
template <typename ElementType, typename IndexType = int, typename LayoutPolicy = layout_c_contiguous>
using host_vector_view = host_mdspan<ElementType, vector_extent<IndexType>, LayoutPolicy>;
template <typename ElementType, typename IndexType = int, typename LayoutPolicy = layout_c_contiguous>
using host_matrix_view = host_mdspan<ElementType, matrix_extent<IndexType>, LayoutPolicy>;

template <typename ElementType, typename IndexType = int>
constexpr auto make_host_scalar_view(ElementType* ptr)
{
  return host_scalar_view<ElementType, IndexType>{ptr, scalar_extent<IndexType>{}};
}
template <typename ElementType, typename IndexType = int, typename LayoutPolicy = layout_c_contiguous>
constexpr auto make_host_vector_view(ElementType* ptr, IndexType n)
{
  return host_vector_view<ElementType, IndexType, LayoutPolicy>{ptr, n};
}
template <typename ElementType, typename IndexType = int, typename LayoutPolicy = layout_c_contiguous>
constexpr auto make_host_matrix_view(ElementType* ptr, IndexType n_rows, IndexType n_cols)
{
  return host_matrix_view<ElementType, IndexType, LayoutPolicy>{
    ptr, matrix_extent<IndexType>{n_rows, n_cols}};
}

}  // namespace raft
