// Cartesian products of parameter lists for test grids (util/itertools.hpp in the
// reference): product<S>({a...}, {b...}, ...) builds S{a_i, b_j, ...} for every
// combination, the last list varying fastest.
#pragma once

#include <initializer_list>
#include <tuple>
#include <utility>
#include <vector>

namespace raft::util::itertools {
namespace detail {
template <typename S, typename... Args, typename T>
void extend(std::vector<S>& out, const std::tuple<Args...>& prefix, const std::vector<T>& last)
{
  for (const auto& v : last)
    out.push_back(std::apply([&](const auto&... p) { return S{p..., v}; }, prefix));
}
template <typename S, typename... Args, typename T, typename... Rest>
void extend(std::vector<S>& out,
            const std::tuple<Args...>& prefix,
            const std::vector<T>& head,
            const std::vector<Rest>&... rest)
{
  for (const auto& v : head)
    extend<S>(out, std::tuple_cat(prefix, std::make_tuple(v)), rest...);
}
}  // namespace detail

template <typename S, typename... Ts>
std::vector<S> product(std::initializer_list<Ts>... lists)
{
  std::vector<S> out;
  detail::extend<S>(out, std::tuple<>{}, std::vector<Ts>(lists)...);
  return out;
}
}  // namespace raft::util::itertools
