#pragma once
#include <raft/core/mdspan_types.hpp>

namespace raft {
// Same view, const elements (core/mdspan.hpp:412 in the reference).
template <typename ElementType, typename Extents, typename Layout>
constexpr auto make_const_mdspan(mdspan<ElementType, Extents, Layout> m)
{
  return mdspan<std::add_const_t<ElementType>, Extents, Layout>(m);
}
}  // namespace raft
