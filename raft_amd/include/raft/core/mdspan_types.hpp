// A minimal multi-dimensional view for the reduction API: what the reference
// takes from libcu++'s mdspan (core/mdspan_types.hpp:10-37, core/mdspan.hpp),
// reduced to ranks 0..2 with run-time extents and the three layouts the path
// can meet: row-major, column-major and strided.
#pragma once

#include <array>
#include <cstddef>
#include <cstdint>
#include <type_traits>

namespace raft {

struct layout_right {};   // C-contiguous: last index fastest
struct layout_left {};    // Fortran-contiguous: first index fastest
struct layout_stride {};  // explicit strides
using layout_c_contiguous = layout_right;
using layout_f_contiguous = layout_left;
using row_major           = layout_right;
using col_major           = layout_left;

template <typename IndexType, size_t Rank>
struct extents {
  using index_type = IndexType;
  static constexpr size_t rank() { return Rank; }
  std::array<IndexType, Rank == 0 ? 1 : Rank> e{};
  constexpr extents() = default;
  template <typename... I, typename = std::enable_if_t<sizeof...(I) == Rank && (Rank > 0)>>
  constexpr extents(I... v) : e{static_cast<IndexType>(v)...}
  {
  }
  constexpr IndexType extent(size_t i) const { return e[i]; }
};
template <typename IndexType>
using scalar_extent = extents<IndexType, 0>;
template <typename IndexType>
using vector_extent = extents<IndexType, 1>;
template <typename IndexType>
using matrix_extent = extents<IndexType, 2>;

template <typename ElementType, typename Extents, typename LayoutPolicy = layout_c_contiguous>
class mdspan {
 public:
  using element_type     = ElementType;
  using value_type       = std::remove_cv_t<ElementType>;
  using extents_type     = Extents;
  using index_type       = typename Extents::index_type;
  using layout_type      = LayoutPolicy;
  using data_handle_type = ElementType*;
  using size_type        = std::make_unsigned_t<index_type>;

  constexpr mdspan() = default;
  constexpr mdspan(ElementType* p, Extents ext) : ptr_(p), ext_(ext) { default_strides(); }
  template <typename I, size_t R = Extents::rank(), typename = std::enable_if_t<R == 1>>
  constexpr mdspan(ElementType* p, I n) : ptr_(p), ext_(n)
  {
    default_strides();
  }
  constexpr mdspan(ElementType* p, Extents ext, std::array<index_type, 2> strides)
    : ptr_(p), ext_(ext), stride_(strides)
  {
  }
  // view of mutable elements -> view of const elements
  template <typename Other,
            typename = std::enable_if_t<std::is_same_v<const Other, ElementType> &&
                                        !std::is_const_v<Other>>>
  constexpr mdspan(const mdspan<Other, Extents, LayoutPolicy>& o)
    : ptr_(o.data_handle()), ext_(o.extents()), stride_{o.stride(0), o.stride(1)}
  {
  }

  static constexpr size_t rank() { return Extents::rank(); }
  constexpr ElementType* data_handle() const { return ptr_; }
  constexpr Extents extents() const { return ext_; }
  constexpr index_type extent(size_t i) const { return ext_.extent(i); }
  constexpr index_type stride(size_t i) const { return stride_[i]; }
  constexpr size_type size() const
  {
    size_type n = 1;
    for (size_t i = 0; i < rank(); ++i)
      n *= static_cast<size_type>(ext_.extent(i));
    return n;
  }
  constexpr bool empty() const { return size() == 0; }
  constexpr bool is_exhaustive() const
  {
    if constexpr (!std::is_same_v<LayoutPolicy, layout_stride>) {
      return true;
    } else if constexpr (Extents::rank() < 2) {
      return Extents::rank() == 0 || stride_[0] == 1;
    } else {
      return (stride_[1] == 1 && stride_[0] == ext_.extent(1)) ||
             (stride_[0] == 1 && stride_[1] == ext_.extent(0));
    }
  }
  // host-side addressing only: the data lives in device memory
  template <typename... I>
  constexpr size_t offset(I... idx) const
  {
    static_assert(sizeof...(I) == Extents::rank());
    const index_type ii[] = {static_cast<index_type>(idx)..., 0};
    size_t off            = 0;
    for (size_t k = 0; k < rank(); ++k)
      off += static_cast<size_t>(ii[k]) * static_cast<size_t>(stride_[k]);
    return off;
  }

 private:
  constexpr void default_strides()
  {
    if constexpr (Extents::rank() == 1) {
      stride_ = {1, 0};
    } else if constexpr (Extents::rank() == 2) {
      if constexpr (std::is_same_v<LayoutPolicy, layout_left>) {
        stride_ = {1, ext_.extent(0)};
      } else {
        stride_ = {ext_.extent(1), 1};
      }
    }
  }
  ElementType* ptr_ = nullptr;
  Extents ext_{};
  std::array<index_type, 2> stride_{0, 0};
};

}  // namespace raft
