#pragma once
#include <raft/core/mdspan_types.hpp>

namespace raft {
// Same view, const elements (core/mdspan.hpp:412 in the reference).
template <typename ElementType, typename Extents, typename Layout>
constexpr auto make_const_mdspan(mdspan<ElementType, Extents, Layout> m)
{
  return mdspan<std::add_const_t<ElementType>, Extents, Layout>(m);
}

// Is T one of this header's views? (the role of is_mdspan_v, core/mdspan.hpp:60-85)
template <typename T>
struct is_mdspan : std::false_type {};
template <typename ElementType, typename Extents, typename Layout>
struct is_mdspan<mdspan<ElementType, Extents, Layout>> : std::true_type {};
template <typename T>
inline constexpr bool is_mdspan_v = is_mdspan<std::remove_cv_t<std::remove_reference_t<T>>>::value;
}  // namespace raft
