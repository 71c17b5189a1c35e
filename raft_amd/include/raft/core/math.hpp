// Host-side raft::abs / min / max / sqrt used by the functor vocabulary.
// Floating min / max ignore NaN, matching what the reference's device
// overloads compute (core/math.hpp:375-397,517-533) and what the kernels do.
#pragma once

#include <cmath>
#include <type_traits>

#include <raft/core/detail/macros.hpp>

namespace raft {

template <typename T>
RAFT_INLINE_FUNCTION auto abs(T x)
{
  if constexpr (std::is_floating_point_v<T>) {
    return std::fabs(x);
  } else if constexpr (std::is_signed_v<T>) {
    return x < T(0) ? T(-x) : x;
  } else {
    return x;
  }
}

template <typename T>
RAFT_INLINE_FUNCTION auto sqrt(T x)
{
  return std::sqrt(x);
}

template <typename T>
RAFT_INLINE_FUNCTION T max(T a, T b)
{
  if constexpr (std::is_floating_point_v<T>) {
    return std::fmax(a, b);
  } else {
    return a < b ? b : a;
  }
}
template <typename T>
RAFT_INLINE_FUNCTION T min(T a, T b)
{
  if constexpr (std::is_floating_point_v<T>) {
    return std::fmin(a, b);
  } else {
    return b < a ? b : a;
  }
}
template <typename T1, typename T2>
RAFT_INLINE_FUNCTION auto max(T1 a, T2 b)
{
  using C = std::common_type_t<T1, T2>;
  return raft::max<C>(static_cast<C>(a), static_cast<C>(b));
}
template <typename T1, typename T2>
RAFT_INLINE_FUNCTION auto min(T1 a, T2 b)
{
  using C = std::common_type_t<T1, T2>;
  return raft::min<C>(static_cast<C>(a), static_cast<C>(b));
}

}  // namespace raft
