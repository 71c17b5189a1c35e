// Layout predicates used by the reduction API's precondition checks
// (util/input_validation.hpp:11-33 in the reference).
#pragma once

#include <raft/core/mdspan_types.hpp>

namespace raft {

template <class T, class E, class L>
constexpr bool is_row_major(mdspan<T, E, L> m)
{
  if constexpr (std::is_same_v<L, layout_right>) {
    return true;
  } else if constexpr (std::is_same_v<L, layout_stride>) {
    return m.stride(1) == typename E::index_type(1) && m.stride(0) >= m.extent(1);
  } else {
    return false;
  }
}

template <class T, class E, class L>
constexpr bool is_col_major(mdspan<T, E, L> m)
{
  if constexpr (std::is_same_v<L, layout_left>) {
    return true;
  } else if constexpr (std::is_same_v<L, layout_stride>) {
    return m.stride(0) == typename E::index_type(1) && m.stride(1) >= m.extent(0);
  } else {
    return false;
  }
}

template <class T, class E, class L>
constexpr bool is_row_or_column_major(mdspan<T, E, L> m)
{
  return is_row_major(m) || is_col_major(m);
}

}  // namespace raft
